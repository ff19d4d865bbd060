"""Novorax on the GPU against the float64 restatement in tests/novorax_ref.py (which processes whole sequences, with no cache,
no state hand-over and no batching): every mechanism alone, prompts against token-by-token decoding, portions down to two
tokens, mixed batches, cells and state slots that are used again, window edges and far memory made loud on purpose, odd sizes,
the serving precision, graph replays, the engine's scheduler and the trace replay tool.

The error of a logits row is the root mean square of (got - want) with the mean taken off, over the row's own root mean square.
F32_TOL bounds rows computed with exact_f32 (f32 re-association only); BF16_TOL rows of the serving precision."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import novorax_ref as R
import novorax_synth as S

pytestmark = pytest.mark.gpu
F32_TOL = 5e-5
BF16_TOL = 6e-2
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def row_err(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return float((np.sqrt((d ** 2).mean(-1)) / np.sqrt((w ** 2).mean(-1))).max())


def toks(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


class Rig:
    """A model folder, its weights for the oracle, and contexts of the product on it."""

    def __init__(self, pkg, folder, cfg, seed=0, tweak=None):
        self.cfg, self.W = cfg, S.weights(cfg, seed)
        if tweak:
            tweak(self.W)
        self.dir = S.write(folder, cfg, self.W)
        self.pkg = pkg
        self.model = pkg.Model(self.dir)

    def ctx(self, n_ctx=256, n_seq_max=4, exact=True, n_ubatch=64, graphs=True):
        return self.pkg.Context(self.model, n_ctx=n_ctx, n_batch=max(n_ctx, n_ubatch), n_ubatch=n_ubatch, n_seq_max=n_seq_max, exact_f32=exact, use_graphs=graphs)

    def ref(self, tokens, layers=False):
        out = R.forward(tokens, self.W, self.cfg, layers)
        return (out[0].numpy(), out[1].numpy()) if layers else out.numpy()


def feed(ctx, tokens, start=0, seq=0, want_all=True):
    """One decode call for tokens[start:] of a sequence; returns the logits of every fed position."""
    n = len(tokens)
    assert ctx.decode(tokens, list(range(start, start + n)), seq=[seq] * n, logits=[1] * n if want_all else None) == 0
    return np.stack([ctx.logits(i) for i in range(n)]) if want_all else ctx.logits(-1)[None]


def feed_in_portions(ctx, tokens, sizes, seq=0):
    out, at, k = [], 0, 0
    while at < len(tokens):
        n = min(sizes[k % len(sizes)], len(tokens) - at)
        out.append(feed(ctx, tokens[at:at + n], at, seq))
        at += n
        k += 1
    return np.concatenate(out)


FULL = [S.latent(mlp=S.dense()), S.mlstm(mlp=S.experts()), S.latent(heads=2, dim=16, rot_dim=4, vdim=24, kv_rank=40, q_rank=24, window=5, mlp=S.experts(n=3, top=1)),
        S.mlstm(heads=1, dim=40, vdim=24, mlp=None)]


@pytest.fixture(scope="module")
def full(pkg, tmp_path_factory):
    """Every mechanism in one small model: both mixers, both feed-forwards, a layer without one, a looped span that starts behind the first layer."""
    return Rig(pkg, tmp_path_factory.mktemp("nvx_full"), S.config(FULL, loop=(1, 3, 2)), seed=3)


# ------------------------------------------------------------------------------------------ each mechanism alone
@pytest.mark.parametrize("name,layers,loop", [
    ("latent", [S.latent()], None),
    ("latent_no_window_plain_rope", [S.latent(window=0, scaling=None, rot_dims=4)], None),
    ("mlstm", [S.mlstm()], None),
    ("dense", [S.latent(heads=1, dim=8, rot_dim=2, vdim=8, kv_rank=8, q_rank=8, mlp=S.dense())], None),
    ("experts", [S.mlstm(heads=1, dim=8, vdim=8, mlp=S.experts())], None),
    ("loop", [S.latent(mlp=S.dense()), S.mlstm()], (0, 2, 3)),
])
def test_mechanism_alone_matches_the_restatement(pkg, tmp_path, name, layers, loop):
    rig = Rig(pkg, tmp_path / name, S.config(layers, loop=loop), seed=11)
    t = toks(29, rig.cfg["vocab"], 5)
    want, taps = rig.ref(t, layers=True)
    c = rig.ctx()
    c.enable_taps(True)
    got = feed(c, t)
    for r in range(taps.shape[0]):
        assert np.abs(c.layer_out(r, len(t)) - taps[r]).max() <= 1e-4 * max(1.0, np.abs(taps[r]).max()), (name, r)
    assert row_err(got, want) <= F32_TOL


# ------------------------------------------------------------------------------------------ prompts, single tokens, portions
def test_prompt_equals_token_by_token(full):
    t = toks(45, full.cfg["vocab"], 1)
    want = full.ref(t)
    whole = feed(full.ctx(), t)
    c = full.ctx()
    single = np.concatenate([feed(c, [t[i]], i) for i in range(len(t))])
    assert row_err(whole, want) <= F32_TOL and row_err(single, want) <= F32_TOL
    assert row_err(single, whole) <= F32_TOL


@pytest.mark.parametrize("sizes", [[2], [3, 2, 7], [17, 2, 2, 30], [64, 5], [1, 2, 1, 9]])
def test_portions_of_any_size(full, sizes):
    t = toks(83, full.cfg["vocab"], 2)
    got = feed_in_portions(full.ctx(n_ubatch=32), t, sizes)          # (portions above 32 are cut again inside the engine)
    assert row_err(got, full.ref(t)) <= F32_TOL


def test_long_decoding_after_a_prompt(full):
    t = toks(300, full.cfg["vocab"], 4)
    c = full.ctx(n_ctx=320)
    got = np.concatenate([feed(c, t[:40])] + [feed(c, [t[i]], i) for i in range(40, len(t))])
    assert row_err(got, full.ref(t)) <= F32_TOL


# ------------------------------------------------------------------------------------------ batches, cells and slots used again
def test_unequal_requests_in_one_batch_equal_each_alone(full):
    V = full.cfg["vocab"]
    reqs = [toks(n, V, 20 + i) for i, n in enumerate((37, 9, 61, 1))]
    want = [full.ref(r) for r in reqs]
    c = full.ctx(n_ctx=192, n_ubatch=48)
    at = [0] * len(reqs)
    got = [[] for _ in reqs]
    plan = [(5, 1, 30, 1), (2, 1, 2, 0), (1, 1, 29, 0), (29, 6, 0, 0), (0, 0, 0, 0)]
    while any(at[i] < len(reqs[i]) for i in range(len(reqs))):
        for step in plan:
            tk, ps, sq, owner = [], [], [], []
            for i, n in enumerate(step):
                n = min(n if n else 1, len(reqs[i]) - at[i])
                tk += reqs[i][at[i]:at[i] + n]; ps += list(range(at[i], at[i] + n)); sq += [i] * n; owner += [i] * n
                at[i] += n
            if not tk:
                continue
            assert c.decode(tk, ps, seq=sq, logits=[1] * len(tk)) == 0
            for j, i in enumerate(owner):
                got[i].append(c.logits(j))
    for i in range(len(reqs)):
        assert row_err(np.stack(got[i]), want[i]) <= F32_TOL, i


def test_cells_and_state_slots_are_used_again(full):
    """A context with room for one request at a time: every request takes the cells and the state slot its predecessor gave back."""
    V = full.cfg["vocab"]
    c = full.ctx(n_ctx=64, n_seq_max=2)
    for k in range(5):
        t = toks(50 + k, V, 40 + k)
        got = feed_in_portions(c, t, [13, 2, 21], seq=k % 2)
        assert row_err(got, full.ref(t)) <= F32_TOL, k
        assert c.kv_used() == len(t)
        assert c.kv_seq_rm(k % 2, -1, -1)
        assert c.kv_used() == 0
    # two live requests in a pool that holds just both: one ends, a third takes its place beside the survivor
    a, b, d = toks(30, V, 50), toks(34, V, 51), toks(28, V, 52)
    ga = feed(c, a, 0, 0)
    gb = feed(c, b[:20], 0, 1)
    assert c.kv_seq_rm(0, -1, -1)
    gd = feed(c, d, 0, 0)
    gb = np.concatenate([gb, feed(c, b[20:], 20, 1)])
    for got, t in ((ga, a), (gb, b), (gd, d)):
        assert row_err(got, full.ref(t)) <= F32_TOL


def test_a_recurrent_state_cannot_be_cut_back(full):
    c = full.ctx()
    feed(c, toks(12, full.cfg["vocab"], 1))
    assert not c.kv_seq_rm(0, 5, -1)          # (the scheduler then drops the whole sequence and starts over)
    assert c.kv_seq_rm(0, -1, -1)


# ------------------------------------------------------------------------------------------ edges made loud
def _sharp_window_rig(pkg, folder, window):
    """One latent-attention layer whose softmax is nearly one-hot (a large score scale, a sink far below the scores): a key that enters or leaves the
    window changes the row it belonged to outright, where random weights at the usual scale would spread the loss over many keys."""
    cfg = S.config([S.latent(heads=2, dim=16, rot_dim=4, vdim=16, kv_rank=32, q_rank=16, window=window, scale=3.0)], width=48, vocab=50)
    return Rig(pkg, folder, cfg, seed=9, tweak=lambda W: W["l0.mix.sink"].fill_(-6.0))


@pytest.mark.parametrize("window", [1, 4, 9])
def test_keys_just_inside_and_just_outside_the_window(pkg, tmp_path, window):
    rig = _sharp_window_rig(pkg, tmp_path / f"w{window}", window)
    t = toks(48, rig.cfg["vocab"], 3)
    want = rig.ref(t)
    # the restatement tells a window that is one token off, in either direction, from the right one
    for off in (-1, 1):
        if window + off < 1:
            continue
        other = json.loads(json.dumps(rig.cfg))
        other["layers"][0]["mixer"]["mask"]["size"] = window + off
        assert row_err(R.forward(t, rig.W, other).numpy(), want) > 3e-2
    assert row_err(feed(rig.ctx(), t), want) <= F32_TOL
    for cut in (window - 1, window, window + 1, 20):           # the prompt ends around the window's edge, the rest is decoded token by token
        cut = max(cut, 1)
        c = rig.ctx()
        got = np.concatenate([feed(c, t[:cut])] + [feed(c, [t[i]], i) for i in range(cut, len(t))])
        assert row_err(got, want) <= F32_TOL, cut
    got = feed_in_portions(rig.ctx(), t, [window, 2, window + 1, 3])
    assert row_err(got, want) <= F32_TOL


def test_first_tokens_and_the_sink(pkg, tmp_path):
    """Position 0 sees one key and the sink: a strong sink takes most of the weight there, a missing one would show at once."""
    cfg = S.config([S.latent(window=3, mlp=None)], width=40, vocab=31)
    rig = Rig(pkg, tmp_path / "sink", cfg, seed=2, tweak=lambda W: W["l0.mix.sink"].copy_(torch.tensor([3.0, -2.0, 0.5]).to(torch.bfloat16)))
    t = toks(6, 31, 8)
    want = rig.ref(t)
    assert row_err(feed(rig.ctx(), t), want) <= F32_TOL
    c = rig.ctx()
    assert row_err(np.concatenate([feed(c, [t[i]], i) for i in range(len(t))]), want) <= F32_TOL
    no_sink = dict(rig.W)
    no_sink.pop("l0.mix.sink")
    assert row_err(R.forward(t, no_sink, cfg).numpy()[:3], want[:3]) > 1e-2


def test_a_token_far_back_stays_in_the_matrix_memory(pkg, tmp_path):
    """Forget gates held open and one loud early token: hundreds of steps later the output still depends on it."""
    cfg = S.config([S.mlstm(heads=2, dim=24, vdim=24, gate_cap=15.0)], width=48, vocab=60)

    def tweak(W):
        W["l0.mix.f.b"][:] = 9.0
        W["l0.mix.f"][:] = W["l0.mix.f"] * 0.05
        W["embed"][5] = W["embed"][5] * 5.0

    rig = Rig(pkg, tmp_path / "far", cfg, seed=4, tweak=tweak)
    t = [x if x != 5 else 6 for x in toks(420, 60, 6)]
    t[3] = 5
    want = rig.ref(t)
    other = list(t)
    other[3] = 6
    assert row_err(rig.ref(other)[-5:], want[-5:]) > 1e-3        # the far token matters at the end
    c = rig.ctx(n_ctx=448, n_ubatch=128)
    got = np.concatenate([feed_in_portions(c, t[:390], [128, 3, 100])] + [feed(c, [t[i]], i) for i in range(390, len(t))])
    assert row_err(got, want) <= F32_TOL


# ------------------------------------------------------------------------------------------ other sizes
@pytest.mark.parametrize("name,cfg", [
    ("ones", S.config([S.latent(heads=1, dim=8, rot_dim=2, vdim=8, kv_rank=8, q_rank=8, window=1, mlp=S.experts(n=1, top=1, ff=8)),
                       S.mlstm(heads=1, dim=1, vdim=1, mlp=S.dense(ff=8))], width=8, vocab=9, loop=(0, 1, 1), logit_scale=1.0)),
    ("wide_latent", S.config([S.latent(heads=5, dim=32, rot_dim=16, vdim=48, kv_rank=200, q_rank=100, window=33, rot_dims=8, mlp=S.experts(n=7, top=3, ff=56))], width=136, vocab=301)),
    ("big_recurrence", S.config([S.mlstm(heads=2, dim=144, vdim=200, mlp=S.dense(ff=264))], width=128, vocab=77)),
    ("no_rotation", S.config([S.latent(rot_dim=0, scaling=None, mlp=None)], width=64, vocab=40)),
    ("odd_width", S.config([S.latent(mlp=S.dense(ff=50)), S.mlstm(mlp=S.experts(ff=30))], width=50, vocab=33, loop=(1, 2, 2))),
    # cache rows that are no multiple of 16 bytes (the attention kernel's scalar-load form), a state deeper than 256 rows, more experts than the grouped batch form takes
    ("unaligned_latent", S.config([S.latent(heads=2, dim=10, rot_dim=6, vdim=14, kv_rank=37, q_rank=22, window=6, mlp=S.dense(ff=30))], width=44, vocab=29)),
    ("deep_recurrence", S.config([S.mlstm(heads=1, dim=300, vdim=70, mlp=None)], width=64, vocab=41)),
    ("many_experts", S.config([S.mlstm(heads=2, dim=8, vdim=8, mlp=S.experts(n=70, top=3, ff=16))], width=32, vocab=90)),
])
def test_other_sizes(pkg, tmp_path, name, cfg):
    rig = Rig(pkg, tmp_path / name, cfg, seed=21)
    t = toks(70, cfg["vocab"], 13)
    want = rig.ref(t)
    got = feed_in_portions(rig.ctx(), t, [40, 2, 1, 27])
    assert row_err(got, want) <= F32_TOL


def test_wide_outputs_with_one_to_four_rows(pkg, tmp_path):
    """Projections with thousands of output columns and one to four rows take the four-weight-rows-per-wave form of the weight-stream kernel (head,
    feed-forward, the experts' pair products stay on the per-row form): portions of 1, 3 and 4 tokens in both precisions."""
    cfg = S.config([S.latent(mlp=S.dense(ff=4104)), S.mlstm(mlp=S.experts(n=3, top=2, ff=48))], width=64, vocab=4099)
    rig = Rig(pkg, tmp_path / "wide", cfg, seed=17)
    t = toks(26, cfg["vocab"], 19)
    want = rig.ref(t)
    for exact, tol in ((True, F32_TOL), (False, F32_TOL)):     # (up to 16 rows the activations stay f32 in either precision)
        got = feed_in_portions(rig.ctx(exact=exact), t, [1, 3, 4, 2])
        assert row_err(got, want) <= tol, exact


# ------------------------------------------------------------------------------------------ serving precision, graphs
def row_errs(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)) / np.sqrt((w ** 2).mean(-1))


def test_serving_precision_is_close_and_takes_the_matrix_cores(full):
    """Batches round their activations to bf16 (2^-9 per element, through seven layer runs of a 72-wide model): most rows land within a
    percent or two, a few rows that sit on a steep gate take several times that; single tokens keep f32 activations and stay at F32_TOL."""
    t = toks(96, full.cfg["vocab"], 30)
    want = full.ref(t)
    exact = feed(full.ctx(n_ubatch=128), t)
    bf = feed(full.ctx(exact=False, n_ubatch=128), t)
    e = row_errs(bf, want)
    assert np.median(e) <= 2e-2 and np.percentile(e, 90) <= BF16_TOL and e.max() <= 0.25, (np.median(e), np.percentile(e, 90), e.max())
    assert row_err(bf, exact) > 1e-5                              # (activations were rounded to bf16: another kernel ran)
    c = full.ctx(exact=False)
    single = np.concatenate([feed(c, [t[i]], i) for i in range(len(t))])
    assert row_err(single, want) <= F32_TOL


def test_graph_replays_equal_eager_steps(full):
    t = toks(40, full.cfg["vocab"], 31)
    outs = []
    for graphs in (True, False):
        c = full.ctx(graphs=graphs)
        feed(c, t[:8], want_all=False)
        rows = []
        for i in range(8, len(t)):
            rows.append(feed(c, [t[i]], i, want_all=False)[0])
            if i % 7 == 0:
                c.synchronize()
        outs.append(np.stack(rows))
    assert np.array_equal(outs[0], outs[1])
    assert row_err(outs[0], full.ref(t)[8:]) <= F32_TOL


# ------------------------------------------------------------------------------------------ the engine and the tools
def test_greedy_generation_through_the_engine(pkg, full):
    """loadmodel -> chat completion through the slot scheduler, two requests side by side; the text is decimal token ids."""
    V = full.cfg["vocab"]
    e = pkg.Engine()
    try:
        st, body = e.load_model(llama_model_path=full.dir, model="nvx", ctx_len=256, n_parallel=2, ngl=100, exact_f32=True, user_prompt="", ai_prompt="", system_prompt="")
        assert st["status_code"] == 200 and not st["has_error"], (st, body)
        prompts = [toks(11, V, 60), toks(23, V, 61)]
        n_new = 12

        def greedy(p):
            seq = list(p)
            for _ in range(n_new + 1):
                seq.append(int(np.argmax(full.ref(seq)[-1])))
            return seq[len(p):]

        import threading
        out = [None, None]

        def run(i):
            res = e.chat_completion(model="nvx", messages=[{"role": "user", "content": " ".join(map(str, prompts[i]))}], max_tokens=n_new, temperature=0.0,
                                    repeat_penalty=1.0, frequency_penalty=0.0, presence_penalty=0.0)
            out[i] = res[-1]

        th = [threading.Thread(target=run, args=(i,)) for i in range(2)]
        [x.start() for x in th]
        [x.join() for x in th]
        for i in range(2):
            st, body = out[i]
            assert st["status_code"] == 200 and not st["has_error"], (st, body)
            got = [int(x) for x in body["choices"][0]["message"]["content"].split()]
            want = greedy(prompts[i])
            assert len(got) >= n_new and got[:n_new] == want[:n_new], (got, want)
    finally:
        e.close()


def test_trace_replay_tool(full, tmp_path):
    V = full.cfg["vocab"]
    a, b = toks(21, V, 70), toks(9, V, 71)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:10], "want": [0, 9]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[10:12], "want": []}, {"id": "b", "tokens": b, "want": [8]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[12:], "want": [8, 0]}], "end": ["a"]}]
    for dtype, tol in (("float32", F32_TOL), ("bfloat16", BF16_TOL)):
        out = tmp_path / dtype
        p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", full.dir, "--dtype", dtype, "--out", str(out), "--max-tokens", "64"],
                           input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
        assert p.returncode == 0, p.stderr[-2000:]
        assert [ln for ln in p.stdout.splitlines() if ln.startswith("done")] == ["done 0", "done 1", "done 2"]
        ra, rb = full.ref(a), full.ref(b)
        g0 = np.fromfile(out / "0.f32", "<f4").reshape(-1, V)
        g1 = np.fromfile(out / "1.f32", "<f4").reshape(-1, V)
        g2 = np.fromfile(out / "2.f32", "<f4").reshape(-1, V)
        assert row_err(g0, ra[[0, 9]]) <= tol and row_err(g1, rb[[8]]) <= tol and row_err(g2, ra[[20, 12]]) <= tol
