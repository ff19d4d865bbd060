// novorax.h — the Novorax design as this runtime holds it: a decoder whose layers each pick a token mixer (latent attention with a sliding window and a
// softmax sink, or the mLSTM matrix-memory recurrence) and a feed-forward (dense relu^2, or experts chosen by a token-id table), norms on both sides of every
// sublayer, and an optional span of layers that runs several times with shared weights, re-fed with the embedding output through an input projection.
//
// Read from a folder: config.json (every size and constant) + model.safetensors (bf16 matrices, int32 tables).  Weights stay bf16 on the device; vectors
// (norm weights, biases, sinks, rotary frequency tables) are widened to f32 at load.  A "layer run" is one execution of a layer: a looped layer has one run
// per pass, each with its own cache plane or recurrent state.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

namespace mi355 {

struct BfMat {                      // bf16 rows on the device
    unsigned short *w = nullptr;
    int N = 0, K = 0;               // rows (outputs), row length (inputs)
};

enum { NVX_LATENT = 0, NVX_MLSTM = 1 };
enum { NVX_FF_NONE = 0, NVX_FF_DENSE = 1, NVX_FF_EXPERTS = 2 };

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
};

struct NvxRun {
    int layer = 0;
    int pass = -1;                  // >= 0: first layer of loop pass `pass` (input projection + step vector come first)
    int plane = -1;                 // latent attention: index of this run's cache plane; mlstm: of its state set
};

struct NovoraxModel {
    std::vector<NvxLayer> layers;
    std::vector<NvxRun> runs;
    BfMat embed, head, loop_in;
    float *loop_step = nullptr;     // [times][width]
    float *final_norm = nullptr;
    float logit_scale = 1.0f, eps = 1e-5f;
    int width = 0, n_vocab = 0;
    int n_latent_runs = 0, n_mlstm_runs = 0;
    // largest sizes over the layers (activation buffers)
    int max_down = 0, max_q_rank = 0, max_q = 0, max_qa = 0, max_att = 0, max_proj = 0, max_ff = 0, max_top = 0, max_expert = 0;
};

}  // namespace mi355
