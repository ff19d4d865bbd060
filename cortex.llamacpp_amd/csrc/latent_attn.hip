// latent_attn.hip — attention through a low-rank latent, on the cache's latent rows themselves.
//
// A token's cache row is [c | r]: the RMS-normed latent c (kv_rank floats) and one rotated key part r (rot floats) shared by all heads.  With W_uk folded
// into the query (qa = W_uk_h^T q_h, a per-head product of mmb.hip) a head's score against a cell is one dot product of length kv_rank + rot,
//   s = (qa . c + rope(q_rot) . r) * scale,
// and the attended value is the weighted sum of latents, unfolded through W_uv afterwards - keys and values are never materialised, every head reads the
// same row.  Visibility: same sequence, 0 <= pos_query - pos_cell < window (window 0: no limit).  The softmax denominator takes one extra term exp(sink_h),
// a learned per-head logit with neither key nor value behind it.  Everything here is f32: positions, angles, scores, weights, the running sums.
//
// latent_prep: per token, the two RMS norms behind the down-projections (query latent -> cq, key / value latent -> cache row) and the rotation of the
// shared key part into the cache row.  Interleaved pairs (2i, 2i + 1); the per-pair frequency table (YaRN blend included) comes from the host.
#include "kernels.h"

namespace mi355 {

namespace {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ float block_sum_256(float v, float *sh) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
    __syncthreads();
    return sh[0] + sh[1] + sh[2] + sh[3];
}

__global__ __launch_bounds__(256) void latent_prep_kernel(LatentPrepArgs a) {
    __shared__ float sh[4];
    const int t = blockIdx.x, tid = threadIdx.x;
    const float *row = a.a + (size_t)t * a.ld_a;
    // query latent
    float ss = 0.0f;
    for (int i = tid; i < a.q_rank; i += 256) { const float v = row[i]; ss = fmaf(v, v, ss); }
    ss = block_sum_256(ss, sh);
    float inv = 1.0f / sqrtf(ss / (float)a.q_rank + a.eps);
    for (int i = tid; i < a.q_rank; i += 256) a.cq[(size_t)t * a.q_rank + i] = row[i] * inv * a.wq_norm[i];
    // key / value latent -> cache row
    const float *kv = row + a.q_rank;
    float *dst = a.cache + (size_t)a.tok_cell[t] * (a.kv_rank + a.rot);
    ss = 0.0f;
    for (int i = tid; i < a.kv_rank; i += 256) { const float v = kv[i]; ss = fmaf(v, v, ss); }
    ss = block_sum_256(ss, sh);
    inv = 1.0f / sqrtf(ss / (float)a.kv_rank + a.eps);
    for (int i = tid; i < a.kv_rank; i += 256) dst[i] = kv[i] * inv * a.wkv_norm[i];
    // shared rotated key part
    const float *kr = kv + a.kv_rank;
    const float p = (float)a.tok_pos[t];
    for (int i = tid; i < a.rot; i += 256) {
        if (i < a.rot_dims) {
            const int pr = i >> 1;
            const float ang = p * a.rot_freq[pr], c = cosf(ang) * a.rot_mscale, s = sinf(ang) * a.rot_mscale;
            const float u = kr[2 * pr], v = kr[2 * pr + 1];
            dst[a.kv_rank + i] = (i & 1) ? v * c + u * s : u * c - v * s;
        } else dst[a.kv_rank + i] = kr[i];
    }
}

constexpr int LA_MAX_ACC = 16;                                  // latent values per lane: kv_rank <= 1024

// one workgroup per (token, head); its four waves take every fourth cell of the scanned range and keep their own running maximum, sum and weighted latent,
// merged at the end together with the sink term
__global__ __launch_bounds__(256) void latent_attn_kernel(LatentAttnArgs a) {
    extern __shared__ float lds[];
    const int KR = a.kv_rank, R = a.rot, L = KR + R;
    float *qv = lds;                                            // [L]
    float *wm = lds + L, *wl = wm + 4, *wacc = wl + 4;           // [4], [4], [4][KR]
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int tpos = a.tok_pos[t];
    const uint64_t sbit = 1ull << (a.tok_seq[t] & 63);
    for (int i = tid; i < KR; i += 256) qv[i] = a.qa[(size_t)t * a.ld_qa + (size_t)h * KR + i];
    {
        const float *qr = a.q + (size_t)t * a.ld_q + (size_t)h * (a.dim + R) + a.dim;
        const float p = (float)tpos;
        for (int i = tid; i < R; i += 256) {
            if (i < a.rot_dims) {
                const int pr = i >> 1;
                const float ang = p * a.rot_freq[pr], c = cosf(ang) * a.rot_mscale, s = sinf(ang) * a.rot_mscale;
                const float u = qr[2 * pr], v = qr[2 * pr + 1];
                qv[KR + i] = (i & 1) ? v * c + u * s : u * c - v * s;
            } else qv[KR + i] = qr[i];
        }
    }
    __syncthreads();
    const int nacc = (KR + 63) >> 6, nall = (L + 63) >> 6;
    float acc[LA_MAX_ACC];
#pragma unroll
    for (int j = 0; j < LA_MAX_ACC; j++) acc[j] = 0.0f;
    float m = -INFINITY, l = 0.0f;
    const int n_kv = *a.n_kv_dev;
    for (int c = wave; c < n_kv; c += 4) {
        const int cp = a.cell_pos[c];
        if (cp < 0 || cp > tpos || !(a.cell_seq[c] & sbit) || (a.window > 0 && tpos - cp >= a.window)) continue;   // (wave-uniform)
        const float *row = a.cache + (size_t)c * L;
        float vals[LA_MAX_ACC], dot = 0.0f;
#pragma unroll
        for (int j = 0; j < LA_MAX_ACC; j++) {
            vals[j] = 0.0f;
            if (j < nacc && j * 64 + lane < KR) { vals[j] = row[j * 64 + lane]; dot = fmaf(vals[j], qv[j * 64 + lane], dot); }
        }
        for (int i = KR + lane; i < L; i += 64) dot = fmaf(row[i], qv[i], dot);
        (void)nall;
        const float s = wave_sum(dot) * a.scale;
        const float mn = fmaxf(m, s), alpha = expf(m - mn), p = expf(s - mn);   // (m = -inf at the first visible cell: alpha = 0)
        l = l * alpha + p;
#pragma unroll
        for (int j = 0; j < LA_MAX_ACC; j++) acc[j] = acc[j] * alpha + p * vals[j];
        m = mn;
    }
    if (lane == 0) { wm[wave] = m; wl[wave] = l; }
#pragma unroll
    for (int j = 0; j < LA_MAX_ACC; j++)
        if (j < nacc && j * 64 + lane < KR) wacc[wave * KR + j * 64 + lane] = acc[j];
    __syncthreads();
    float M = fmaxf(fmaxf(wm[0], wm[1]), fmaxf(wm[2], wm[3]));
    const float sink = a.sink ? a.sink[h] : -INFINITY;
    M = fmaxf(M, sink);
    float sc[4], den = a.sink ? expf(sink - M) : 0.0f;
#pragma unroll
    for (int w = 0; w < 4; w++) { sc[w] = wl[w] > 0.0f ? expf(wm[w] - M) : 0.0f; den += wl[w] * sc[w]; }
    const float inv = den > 0.0f ? 1.0f / den : 0.0f;
    for (int i = tid; i < KR; i += 256) {
        const float o = wacc[i] * sc[0] + wacc[KR + i] * sc[1] + wacc[2 * KR + i] * sc[2] + wacc[3 * KR + i] * sc[3];
        a.out[(size_t)t * a.ld_out + (size_t)h * KR + i] = o * inv;
    }
}

}  // namespace

bool latent_attn_shape_ok(int kv_rank, int rot) { return kv_rank >= 1 && kv_rank <= 64 * LA_MAX_ACC && rot >= 0 && rot <= 4096; }

hipError_t launch_latent_prep(const LatentPrepArgs &a, hipStream_t st) {
    if (a.T <= 0) return hipSuccess;
    if (a.rot_dims > a.rot || (a.rot_dims & 1)) return hipErrorInvalidValue;
    hipLaunchKernelGGL(latent_prep_kernel, dim3((unsigned)a.T), dim3(256), 0, st, a);
    return hipGetLastError();
}

hipError_t launch_latent_attn(const LatentAttnArgs &a, hipStream_t st) {
    if (a.T <= 0) return hipSuccess;
    if (!latent_attn_shape_ok(a.kv_rank, a.rot) || a.rot_dims > a.rot || (a.rot_dims & 1)) return hipErrorInvalidValue;
    const size_t lds = (size_t)(a.kv_rank + a.rot + 8 + 4 * a.kv_rank) * sizeof(float);
    hipLaunchKernelGGL(latent_attn_kernel, dim3((unsigned)a.T, (unsigned)a.H), dim3(256), lds, st, a);
    return hipGetLastError();
}

}  // namespace mi355
