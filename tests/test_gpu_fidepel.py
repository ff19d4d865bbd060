"""Fidepel on the GPU against the float64 restatement in tests/fidepel_ref.py (which processes whole sequences, with no cache and no batching):
every mechanism alone, prompts against token-by-token decoding, portions down to two tokens, mixed batches, cells and sequence slots that are used
again, window edges and far keys made loud on purpose, first tokens, long decoding, odd sizes, the serving precision, graph replays, the engine's
scheduler and the trace replay tool.

The error of a logits row is the root mean square of (got - want) with the mean taken off, over the row's own root mean square.
F32_TOL bounds rows computed with exact_f32 (f32 re-association only); BF16_TOL rows of the serving precision."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import fidepel_ref as R
import fidepel_synth as S

pytestmark = pytest.mark.gpu
F32_TOL = 5e-5
BF16_TOL = 6e-2
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def row_errs(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)) / np.sqrt((w ** 2).mean(-1))


def row_err(got, want):
    return float(row_errs(got, want).max())


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

    def ref(self, tokens, layers=False, cfg=None):
        out = R.forward(tokens, self.W, cfg or self.cfg, layers)
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


def one_by_one(ctx, tokens, start=0, seq=0):
    return np.concatenate([feed(ctx, [tokens[i]], i, seq) for i in range(start, len(tokens))])


FULL = [S.attention(mlp=S.moe()),
        S.attention(heads=4, kv_heads=4, dim=12, vdim=12, window=5, rot_dims=12, factor=None, mlp=S.moe(n=5, top=1, ff=24, groups=None, shared=0)),
        S.attention(heads=3, kv_heads=1, dim=20, vdim=36, window=0, rot_dims=0, mlp=None),
        S.attention(heads=2, kv_heads=1, dim=16, vdim=8, window=11, rot_dims=4, mlp=S.moe(n=8, top=3, ff=16, groups=(4, 3), shared=56))]


@pytest.fixture(scope="module")
def full(pkg, tmp_path_factory):
    """Every branch in one small model: grouped and ungrouped routing, with and without the shared expert, a block without a feed-forward, windows and none,
    rotation of the whole head, of a part and none, one to several key heads, a looped span in the middle."""
    return Rig(pkg, tmp_path_factory.mktemp("fdp_full"), S.config(FULL, loop=(1, 3, 2)), seed=3)


# ------------------------------------------------------------------------------------------ each mechanism alone
@pytest.mark.parametrize("name,layers,loop", [
    ("attention", [S.attention()], None),
    ("attention_whole_head_turns_no_scaling", [S.attention(rot_dims=24, factor=None)], None),
    ("attention_no_rotation_no_window", [S.attention(rot_dims=0, window=0)], None),
    ("attention_every_head_its_own_key", [S.attention(heads=3, kv_heads=3)], None),
    ("router_plain", [S.attention(heads=1, kv_heads=1, dim=8, vdim=8, rot_dims=2, mlp=S.moe(groups=None, shared=0))], None),
    ("router_groups", [S.attention(heads=1, kv_heads=1, dim=8, vdim=8, rot_dims=2, mlp=S.moe(n=12, top=3, groups=(4, 2), shared=0))], None),
    ("shared_expert", [S.attention(heads=1, kv_heads=1, dim=8, vdim=8, rot_dims=2, mlp=S.moe(n=2, top=1, groups=None, shared=40))], None),
    ("loop", [S.attention(mlp=S.moe()), S.attention(heads=2, kv_heads=1, dim=8, vdim=8, rot_dims=8)], (0, 2, 3)),
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


def test_the_router_takes_the_restatements_experts(pkg, tmp_path):
    """Group limits bite: with a strong router the best expert overall often sits in a group that another group's best member closes.  A router that ignored
    the groups, or the `keep` count, or the weights' scale, would miss the restatement by far more than the tolerance."""
    mlp = S.moe(n=12, top=2, ff=24, groups=(3, 1), scale=2.5, shared=0)
    cfg = S.config([S.attention(heads=1, kv_heads=1, dim=8, vdim=8, rot_dims=4, mlp=mlp)], width=40, vocab=61)
    rig = Rig(pkg, tmp_path / "groups", cfg, seed=5)
    t = toks(40, 61, 6)
    want = rig.ref(t)
    for change in ({"groups": None}, {"groups": {"count": 3, "keep": 2}}, {"scale": 1.0}):
        other = json.loads(json.dumps(cfg))
        for k, v in change.items():
            if v is None:
                other["layers"][0]["mlp"]["router"].pop(k)
            else:
                other["layers"][0]["mlp"]["router"][k] = v
        assert row_err(rig.ref(t, cfg=other), want) > 1e-2, change
    assert row_err(feed(rig.ctx(), t), want) <= F32_TOL
    assert row_err(one_by_one(rig.ctx(), t), want) <= F32_TOL


# ------------------------------------------------------------------------------------------ prompts, single tokens, portions
def test_prompt_equals_token_by_token(full):
    t = toks(45, full.cfg["vocab"], 1)
    want = full.ref(t)
    whole = feed(full.ctx(), t)
    single = one_by_one(full.ctx(), t)
    assert row_err(whole, want) <= F32_TOL and row_err(single, want) <= F32_TOL
    assert row_err(single, whole) <= F32_TOL


@pytest.mark.parametrize("sizes", [[2], [3, 2, 7], [17, 2, 2, 30], [64, 5], [1, 2, 1, 9], [12, 11, 13]])
def test_portions_of_any_size(full, sizes):
    t = toks(83, full.cfg["vocab"], 2)
    got = feed_in_portions(full.ctx(n_ubatch=32), t, sizes)          # (portions above 32 are cut again inside the engine)
    assert row_err(got, full.ref(t)) <= F32_TOL


def test_long_decoding_after_a_prompt(full):
    t = toks(300, full.cfg["vocab"], 4)
    c = full.ctx(n_ctx=320)
    got = np.concatenate([feed(c, t[:40]), one_by_one(c, t, 40)])
    assert row_err(got, full.ref(t)) <= F32_TOL


def test_the_first_tokens_of_a_sequence(full):
    """Position 0 sees one key, position 1 two: every softmax of the first rows is short, and the windows have not filled yet."""
    t = toks(4, full.cfg["vocab"], 9)
    want = full.ref(t)
    assert row_err(feed(full.ctx(), t), want) <= F32_TOL
    assert row_err(one_by_one(full.ctx(), t), want) <= F32_TOL
    assert row_err(feed_in_portions(full.ctx(), t, [1, 3]), want) <= F32_TOL
    assert row_err(feed(full.ctx(), t[:1]), want[:1]) <= F32_TOL


# ------------------------------------------------------------------------------------------ batches, cells and slots used again
def test_unequal_requests_in_one_batch_equal_each_alone(full):
    V = full.cfg["vocab"]
    reqs = [toks(n, V, 20 + i) for i, n in enumerate((37, 9, 61, 1))]
    want = [full.ref(r) for r in reqs]
    c = full.ctx(n_ctx=192, n_ubatch=48)                     # (48 cells per sequence region: the 61-token request spills into its neighbours')
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


def test_cells_and_sequence_slots_are_used_again(full):
    """A context with room for one request at a time: every request takes the cells its predecessor gave back; then two live requests in a pool that holds
    just both, one ends and a third takes its place beside the survivor."""
    V = full.cfg["vocab"]
    c = full.ctx(n_ctx=64, n_seq_max=2)
    for k in range(5):
        t = toks(50 + k, V, 40 + k)
        got = feed_in_portions(c, t, [13, 2, 21], seq=k % 2)
        assert row_err(got, full.ref(t)) <= F32_TOL, k
        assert c.kv_used() == len(t)
        assert c.kv_seq_rm(k % 2, -1, -1)
        assert c.kv_used() == 0
    a, b, d = toks(30, V, 50), toks(34, V, 51), toks(28, V, 52)
    ga = feed(c, a, 0, 0)
    gb = feed(c, b[:20], 0, 1)
    assert c.kv_seq_rm(0, -1, -1)
    gd = feed(c, d, 0, 0)
    gb = np.concatenate([gb, feed(c, b[20:], 20, 1)])
    for got, t in ((ga, a), (gb, b), (gd, d)):
        assert row_err(got, full.ref(t)) <= F32_TOL


def test_a_sequence_cut_back_is_decoded_again(full):
    """Pure attention keeps nothing but its cells: the tail of a sequence can be dropped and fed again (what a scheduler does with a shared prefix)."""
    t = toks(30, full.cfg["vocab"], 7)
    c = full.ctx()
    feed(c, t)
    assert c.kv_seq_rm(0, 12, -1)
    got = feed(c, t[12:], 12)
    assert row_err(got, full.ref(t)[12:]) <= F32_TOL


# ------------------------------------------------------------------------------------------ edges made loud
def _sharp_rig(pkg, folder, window, seed=9, tweak_weights=None, **kw):
    """One attention block whose softmax is nearly one-hot (a large score scale): a key that enters or leaves the window changes the row it belonged to
    outright, where random weights at the usual scale would spread the loss over many keys."""
    cfg = S.config([S.attention(heads=2, kv_heads=1, dim=16, vdim=16, window=window, rot_dims=8, scale=2.0, **kw)], width=48, vocab=50)
    return Rig(pkg, folder, cfg, seed=seed, tweak=tweak_weights)


@pytest.mark.parametrize("window", [1, 4, 9])
def test_keys_just_inside_and_just_outside_the_window(pkg, tmp_path, window):
    rig = _sharp_rig(pkg, tmp_path / f"w{window}", window)
    t = toks(48, rig.cfg["vocab"], 3)
    want = rig.ref(t)
    # the restatement tells a window that is one token off, in either direction, from the right one
    for off in (-1, 1):
        if window + off < 1:
            continue
        other = json.loads(json.dumps(rig.cfg))
        other["layers"][0]["mixer"]["mask"]["size"] = window + off
        assert row_err(rig.ref(t, cfg=other), want) > 3e-2
    assert row_err(feed(rig.ctx(), t), want) <= F32_TOL
    for cut in (window - 1, window, window + 1, 20):           # the prompt ends around the window's edge, the rest is decoded token by token
        cut = max(cut, 1)
        c = rig.ctx()
        got = np.concatenate([feed(c, t[:cut]), one_by_one(c, t, cut)])
        assert row_err(got, want) <= F32_TOL, cut
    got = feed_in_portions(rig.ctx(), t, [window, 2, window + 1, 3])
    assert row_err(got, want) <= F32_TOL


def _loud_rig(pkg, folder, window, gain=6.0, d0=12, seed=4):
    """The sharp block with one unrotated coordinate of every query and key made loud through the norm weights: the score is then decided by that coordinate."""
    def tweak(W):
        for h in range(2):
            W["l0.mix.q.norm"][h * 16 + d0] *= gain
        W["l0.mix.k.norm"][d0] *= gain
    return _sharp_rig(pkg, folder, window, seed=seed, tweak_weights=tweak)


def _loud_sequence(rig, n, p0, askers, d0=12, seed=6):
    """n tokens whose keys are quiet in the loud coordinate, except ONE token at position p0 whose key is the loudest of the vocabulary; the rows in `askers`
    hold the quiet token whose query asks for it most.  While p0 is inside an asker's window that key takes nearly all of its weight."""
    F64, W, eps = torch.float64, rig.W, rig.cfg["norm"]["eps"]
    h = R.norm_one_number(W["embed"].to(F64), W["l0.norm1"], eps)
    k = (R.unit(h @ W["l0.mix.k"].to(F64).T, eps) * W["l0.mix.k.norm"].to(F64))[:, d0]
    q = (R.unit(h @ W["l0.mix.q"].to(F64).T, eps) * W["l0.mix.q.norm"].to(F64))[:, d0] * W["l0.mix.temp"].to(F64)[0]
    loud = int(torch.argmax(k))
    quiet = [int(i) for i in torch.argsort(k.abs()) if int(i) != loud][:30]
    asker = max(quiet, key=lambda i: float(q[i]))
    t = [quiet[int(i)] for i in torch.randint(0, len(quiet), (n,), generator=torch.Generator().manual_seed(seed))]
    t[p0] = loud
    for r in askers:
        t[r] = asker
    return t


@pytest.mark.parametrize("window,p0", [(300, 10), (300, 100), (64, 3), (129, 63)])
def test_a_far_key_at_the_windows_edge(pkg, tmp_path, window, p0):
    """One loud key hundreds of positions back: the row at distance window - 1 still sees it (and gives it nearly all its weight), the next row has lost it.
    The restatement with a window one token off changes exactly one of the two rows outright.  Checked for whole prompts, for portions whose micro-batches
    end between the key and the edge, for single tokens across the edge, and with the sequence's cells crossing its region's border (regions of
    n_ctx / 4 cells)."""
    rig = _loud_rig(pkg, tmp_path / "loud", window)
    r_in, r_out = p0 + window - 1, p0 + window
    n = r_out + 20
    t = _loud_sequence(rig, n, p0, [r_in, r_out])
    want = rig.ref(t)
    for w, row in ((window - 1, r_in), (window + 1, r_out)):
        other = json.loads(json.dumps(rig.cfg))
        other["layers"][0]["mixer"]["mask"]["size"] = w
        e = row_errs(rig.ref(t, cfg=other), want)
        assert e[row] > 0.3 and e[r_in + r_out - row] < 1e-3, (w, e[r_in], e[r_out])
    n_ctx = (n + 63) // 64 * 64
    assert row_err(feed(rig.ctx(n_ctx=n_ctx, n_ubatch=512), t), want) <= F32_TOL
    c = rig.ctx(n_ctx=n_ctx, n_ubatch=128)
    assert row_err(feed_in_portions(c, t, [r_in, 2, 100]), want) <= F32_TOL          # the edge is the first row of a two-token portion
    c = rig.ctx(n_ctx=n_ctx, n_ubatch=128)
    assert row_err(feed_in_portions(c, t, [r_in + 1, 100]), want) <= F32_TOL          # ... and the last row of a prompt portion
    c = rig.ctx(n_ctx=n_ctx, n_ubatch=128)
    got = np.concatenate([feed_in_portions(c, t[:r_in - 3], [128, 3, 100]), one_by_one(c, t, r_in - 3)])    # single tokens across the edge
    assert row_err(got, want) <= F32_TOL


def test_window_edges_while_other_requests_come_and_go(pkg, tmp_path):
    """The windowed request decodes token by token while short requests beside it start, end and hand their cells on: its visible cells are then spread
    over cells that were used before, and the scan bounds of every step must still cover exactly its window."""
    rig = _sharp_rig(pkg, tmp_path / "churn", 6)
    V = rig.cfg["vocab"]
    t = toks(70, V, 12)
    want = rig.ref(t)
    c = rig.ctx(n_ctx=64, n_seq_max=4, n_ubatch=16)
    got = [feed(c, t[:5], 0, 0)]
    for i in range(5, len(t)):
        other = toks(3 + i % 4, V, 100 + i)
        slot = 1 + i % 3
        tk = [t[i]] + other
        ps = [i] + list(range(len(other)))
        sq = [0] + [slot] * len(other)
        assert c.decode(tk, ps, seq=sq, logits=[1] * len(tk)) == 0
        got.append(c.logits(0)[None])
        assert row_err(np.stack([c.logits(1 + j) for j in range(len(other))]), rig.ref(other)) <= F32_TOL
        assert c.kv_seq_rm(slot, -1, -1)
        if i % 9 == 0:                                           # now and then the long request gives up cells that lie outside every later window
            assert c.kv_seq_rm(0, 0, i - 8)
    assert row_err(np.concatenate(got), want) <= F32_TOL


# ------------------------------------------------------------------------------------------ other sizes
@pytest.mark.parametrize("name,cfg", [
    ("ones", S.config([S.attention(heads=1, kv_heads=1, dim=2, vdim=1, window=1, rot_dims=2, mlp=S.moe(n=1, top=1, ff=8, groups=(1, 1), shared=1))], width=8, vocab=9,
                      loop=(0, 1, 1), residual_mult=1.0)),
    ("wide_heads", S.config([S.attention(heads=4, kv_heads=2, dim=160, vdim=72, window=33, rot_dims=64, mlp=S.moe(n=7, top=3, ff=56, groups=None, shared=80))], width=136, vocab=301)),
    ("wide_values", S.config([S.attention(heads=2, kv_heads=1, dim=32, vdim=256, window=40, rot_dims=32, mlp=None)], width=64, vocab=77)),
    ("very_wide_heads", S.config([S.attention(heads=2, kv_heads=1, dim=320, vdim=272, window=50, rot_dims=320, mlp=None)], width=96, vocab=55)),
    ("equal_head_sizes", S.config([S.attention(heads=8, kv_heads=4, dim=64, vdim=64, window=16, rot_dims=32, mlp=S.moe(n=16, top=4, ff=32, groups=(8, 4), shared=32))], width=128, vocab=200)),
    # heads whose keys and values do not start on 16-byte boundaries (the attention kernel's scalar-load form), a width that is no multiple of 8
    ("unaligned", S.config([S.attention(heads=3, kv_heads=3, dim=10, vdim=14, window=6, rot_dims=6, mlp=S.moe(n=4, top=2, ff=30, groups=(2, 1), shared=18))], width=44, vocab=29)),
    ("odd_width_loop_tail", S.config([S.attention(mlp=S.moe(ff=30)), S.attention(heads=2, kv_heads=2, dim=6, vdim=6, rot_dims=0, mlp=None), S.attention(mlp=S.moe(shared=0))],
                                     width=50, vocab=33, loop=(1, 3, 3))),
    # more experts than the grouped batch form takes (pair products for batches too), every group kept
    ("many_experts", S.config([S.attention(heads=2, kv_heads=1, dim=8, vdim=8, rot_dims=8, mlp=S.moe(n=70, top=3, ff=16, groups=(7, 7), shared=8))], width=32, vocab=90)),
    ("a_window_wider_than_the_context", S.config([S.attention(window=4000, mlp=S.moe())], width=40, vocab=31)),
])
def test_other_sizes(pkg, tmp_path, name, cfg):
    rig = Rig(pkg, tmp_path / name, cfg, seed=21)
    t = toks(70, cfg["vocab"], 13)
    want = rig.ref(t)
    got = feed_in_portions(rig.ctx(), t, [40, 2, 1, 27])
    assert row_err(got, want) <= F32_TOL


def test_wide_outputs_with_one_to_four_rows(pkg, tmp_path):
    """A head and a shared expert with thousands of output columns and one to four rows take the four-weight-rows-per-wave form of the weight-stream kernel:
    portions of 1, 3 and 4 tokens in both precisions (up to 16 rows the activations stay f32 in either)."""
    cfg = S.config([S.attention(mlp=S.moe(shared=4104))], width=64, vocab=4099)
    rig = Rig(pkg, tmp_path / "wide", cfg, seed=17)
    t = toks(26, cfg["vocab"], 19)
    want = rig.ref(t)
    for exact in (True, False):
        got = feed_in_portions(rig.ctx(exact=exact), t, [1, 3, 4, 2])
        assert row_err(got, want) <= F32_TOL, exact


# ------------------------------------------------------------------------------------------ serving precision, graphs
def test_serving_precision_is_close_and_takes_the_matrix_cores(full):
    """Batches round their activations to bf16 (2^-9 per element, through six layer runs of a 72-wide model): most rows land within a percent or two; a
    token whose router scores lie close picks another expert now and then and takes several times that.  Single tokens keep f32 activations."""
    t = toks(96, full.cfg["vocab"], 30)
    want = full.ref(t)
    exact = feed(full.ctx(n_ubatch=128), t)
    bf = feed(full.ctx(exact=False, n_ubatch=128), t)
    e = row_errs(bf, want)
    assert np.median(e) <= 2e-2 and np.percentile(e, 90) <= BF16_TOL, (np.median(e), np.percentile(e, 90), e.max())
    assert row_err(bf, exact) > 1e-5                              # (activations were rounded to bf16: another kernel ran)
    single = one_by_one(full.ctx(exact=False), t)
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


def test_feed_forward_branches_on_side_streams_change_no_bit(full, monkeypatch):
    """The routed and the shared experts of a block run on side streams beside its attention (forked behind the block projection, joined before the closing
    sum); MI355_BLOCK_FORK=0 keeps every launch on one stream.  Same launches, same order of additions: prompts, portions and replayed single-token steps
    give the same bits either way."""
    t = toks(90, full.cfg["vocab"], 33)
    outs = []
    for fork in ("1", "0"):
        monkeypatch.setenv("MI355_BLOCK_FORK", fork)
        c = full.ctx(n_ubatch=32)
        outs.append(np.concatenate([feed_in_portions(c, t[:60], [40, 3, 17]), one_by_one(c, t, 60)]))
    assert np.array_equal(outs[0], outs[1])
    assert row_err(outs[0], full.ref(t)) <= F32_TOL


# ------------------------------------------------------------------------------------------ the engine and the tools
def test_greedy_generation_through_the_engine(pkg, full):
    """loadmodel -> chat completion through the slot scheduler, two requests side by side; the text is decimal token ids."""
    V = full.cfg["vocab"]
    e = pkg.Engine()
    try:
        st, body = e.load_model(llama_model_path=full.dir, model="fdp", ctx_len=256, n_parallel=2, ngl=100, exact_f32=True, user_prompt="", ai_prompt="", system_prompt="")
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
            res = e.chat_completion(model="fdp", messages=[{"role": "user", "content": " ".join(map(str, prompts[i]))}], max_tokens=n_new, temperature=0.0,
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


def test_trace_tool_with_a_pool_that_is_always_full(pkg, tmp_path):
    """Up to four live requests of unequal lengths fed in portions of changing size beside single tokens of the others, in a pool that holds exactly what
    the live requests need (each rounded up to 64 cells): a finished request's cells and slot go to the next one at once.  Every position of every request
    is asked for and compared with the restatement, in both precisions."""
    cfg = S.config([S.attention(heads=6, kv_heads=3, dim=16, vdim=24, window=21, rot_dims=12, mlp=S.moe(n=9, top=2, ff=24, groups=(3, 2), shared=40)),
                    S.attention(heads=2, kv_heads=1, dim=32, vdim=16, window=70, rot_dims=32, factor=2.0, mlp=S.moe(n=4, top=1, ff=32, groups=None, shared=0)),
                    S.attention(heads=4, kv_heads=4, dim=8, vdim=8, window=0, rot_dims=0, mlp=None)], width=88, vocab=211, loop=(0, 2, 2))
    rig = Rig(pkg, tmp_path / "pool", cfg, seed=31)
    V = cfg["vocab"]
    rng = np.random.default_rng(5)
    lengths = [150, 64, 97, 1, 33, 128, 70, 191, 2, 65]
    reqs = {f"q{i}": toks(n, V, 300 + i) for i, n in enumerate(lengths)}
    waiting, live, at = list(reqs), [], {}
    steps, need = [], 0
    while waiting or live:
        while waiting and len(live) < 4:
            r = waiting.pop(0)
            live.append(r)
            at[r] = 0
        need = max(need, sum((len(reqs[r]) + 63) // 64 * 64 for r in live))
        entries, end = [], []
        for k, r in enumerate(live):
            if len(live) > 1 and rng.random() < 0.2:
                continue                                         # a request may sit a step out
            n = int(rng.choice([1, 1, 1, 2, 3, 5, 17, 40])) if at[r] > 0 or k != 1 else len(reqs[r])
            n = min(n, len(reqs[r]) - at[r])
            entries.append({"id": r, "tokens": reqs[r][at[r]:at[r] + n], "want": list(range(n))})
            at[r] += n
            if at[r] == len(reqs[r]):
                end.append(r)
        steps.append({"step": len(steps), "entries": entries, "end": end})
        live = [r for r in live if r not in end]
    want = {r: rig.ref(t) for r, t in reqs.items()}
    for dtype in ("float32", "bfloat16"):
        out = tmp_path / dtype
        p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", rig.dir, "--dtype", dtype, "--out", str(out), "--max-tokens", str(need)],
                           input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
        assert p.returncode == 0, p.stderr[-2000:]
        got, fed = {r: [] for r in reqs}, {r: 0 for r in reqs}
        for st in steps:
            if not any(e["want"] for e in st["entries"]):
                continue
            rows = np.fromfile(out / f"{st['step']}.f32", "<f4").reshape(-1, V)
            k = 0
            for e in st["entries"]:
                got[e["id"]].append(rows[k:k + len(e["want"])])
                k += len(e["want"])
            assert k == len(rows)
        errs = np.concatenate([row_errs(np.concatenate(got[r]), want[r]) for r in reqs])
        if dtype == "float32":
            assert errs.max() <= F32_TOL, errs.max()
        else:
            assert np.median(errs) <= 2e-2 and np.percentile(errs, 90) <= BF16_TOL, (np.median(errs), np.percentile(errs, 90), errs.max())
