// novorax.h — the layer stack of the folder models (config.json + model.safetensors, bf16 weights) as this runtime holds it.  Two designs fill it.
//
// Novorax: a decoder whose layers each pick a token mixer (latent attention with a sliding window and a
// softmax sink, or the mLSTM matrix-memory recurrence) and a feed-forward (dense relu^2, or experts chosen by a token-id table), norms on both sides of every
// sublayer, and an optional span of layers that runs several times with shared weights, re-fed with the embedding output through an input projection.
//
// Read from a folder: config.json (every size and constant) + model.safetensors (bf16 matrices, int32 tables).  Weights stay bf16 on the device; vectors
// (norm weights, biases, sinks, rotary frequency tables) are widened to f32 at load.  A "layer run" is one execution of a layer: a looped layer has one run
// per pass, each with its own cache plane or recurrent state.
//
// Fidepel: every layer is ONE block - h = norm(x) with a one-number weight, x += m * (mixer(h) + feed_forward(h)) - whose mixer is grouped-query attention
// (RMS norm over the whole query and the whole key projection, rotate-half rotary positions on part of each head with linearly scaled frequencies, a score
// multiplier per head, a sliding window, a sigmoid output gate per head) and whose feed-forward is a routed mixture of relu^2 experts (softmax scores, expert
// groups of which only the best stay open, renormalised and scaled weights) plus an always-on shared expert; a span of layers may run several times with
// shared weights and nothing between the passes.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

namespace mi355 {

struct BfMat {                      // bf16 rows on the device
    unsigned short *w = nullptr;
    int N = 0, K = 0;               // rows (outputs), row length (inputs)
};

enum { NVX_LATENT = 0, NVX_MLSTM = 1, NVX_GQ = 2 };              // token mixers: latent attention, matrix-memory recurrence, grouped-query attention
enum { NVX_FF_NONE = 0, NVX_FF_DENSE = 1, NVX_FF_EXPERTS = 2, NVX_FF_ROUTED = 3 };   // dense; experts by a token-id table; experts by a router

struct NvxLayer {
    int type = NVX_LATENT;
    // mixer sizes (latent attention: all; mlstm: heads, dim, vdim, gate_cap)
    int heads = 0, dim = 0, vdim = 0, rot = 0, kv_rank = 0, q_rank = 0, window = 0, rot_dims = 0;
    float scale = 1.0f, rot_mscale = 1.0f, gate_cap = 1.0f;
    float *rot_freq = nullptr;      // [rot_dims / 2] radians per position
    float *norm1 = nullptr, *norm1b = nullptr, *norm2 = nullptr, *norm2b = nullptr;
    // latent attention: down = [dq ; dkv] rows, uk_t = per head [kv_rank][dim] (W_uk transposed inside each head), uv = per head [vdim][kv_rank]
    BfMat down, uq, uk_t, uv, o;
    float *dq_norm = nullptr, *dkv_norm = nullptr, *sink = nullptr;
    // mlstm: proj = [q ; k ; v ; g ; i ; f] rows
    BfMat proj;
    float *mix_norm = nullptr, *i_bias = nullptr, *f_bias = nullptr;
    // feed-forward
    int ff_kind = NVX_FF_NONE, ff = 0, n_expert = 0, top = 0;
    BfMat up, down_ff;              // dense; experts: gate / up packed [n_expert][ff][width], down packed [n_expert][width][ff]
    BfMat e_gate, e_up, e_down;
    int32_t *table = nullptr;       // [n_vocab][top]
    // grouped-query attention: proj = [q: heads*dim ; k: kv_heads*dim ; v: kv_heads*vdim ; g: heads ; router: n_expert] rows, one product per block
    // (proj above); q_norm / k_norm over the whole projection; head_scale = the per-head score multiplier; the gate and router columns start at off_gate / off_router
    int kv_heads = 0, off_gate = -1, off_router = -1;
    float *q_norm = nullptr, *k_norm = nullptr, *head_scale = nullptr;
    // routed experts (e_up [n_expert][ff][width] with relu^2, e_down [n_expert][width][ff]): groups of neighbouring experts, the `group_keep` best stay open;
    // weights s / sum * router_scale; the shared expert s_up / s_down (shared_ff 0: none) runs for every token
    int n_group = 1, group_keep = 1, shared_ff = 0;
    float router_scale = 1.0f;
    BfMat s_up, s_down;
    int cache_row() const { return type == NVX_LATENT ? kv_rank + rot : type == NVX_GQ ? kv_heads * (dim + vdim) : 0; }   // f32 per cell of a run's cache plane
};

struct NvxRun {
    int layer = 0;
    int pass = -1;                  // >= 0: first layer of loop pass `pass` (input projection + step vector come first)
    int plane = -1;                 // attention mixers: index of this run's cache plane; mlstm: of its state set
};

struct NovoraxModel {
    std::vector<NvxLayer> layers;
    std::vector<NvxRun> runs;
    BfMat embed, head, loop_in;
    float *loop_step = nullptr;     // [times][width]
    float *final_norm = nullptr;
    float logit_scale = 1.0f, eps = 1e-5f;
    std::string design;             // "novorax" | "fidepel"
    // norm weights: the factor is norm_off + w (1: zero-centred weights, 0: plain ones).  parallel_block: one norm per layer, mixer and feed-forward both read
    // it, x += residual_mult * (their sum); otherwise norms on both sides of each sublayer
    float norm_off = 1.0f, residual_mult = 1.0f;
    bool parallel_block = false;
    int width = 0, n_vocab = 0;
    int n_cache_runs = 0, n_mlstm_runs = 0;
    int max_window = 0;             // largest window of the windowed attention layers, 0 if one of them sees every earlier cell (scan bounds)
    int max_shared_ff = 0;
    // largest sizes over the layers (activation buffers)
    int max_down = 0, max_q_rank = 0, max_q = 0, max_qa = 0, max_att = 0, max_proj = 0, max_ff = 0, max_top = 0, max_expert = 0;
};

}  // namespace mi355
