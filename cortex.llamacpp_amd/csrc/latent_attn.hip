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

constexpr int LA_MAX_L = 1088;                                  // kv_rank + rot the attention kernel is instantiated for (17 x 64)

// One workgroup per (token, head), NW waves.  A wave works on four cells at a time: each 16-lane group owns one cell, its lanes hold the row's elements
// 64 j + 4 li .. + 3 (16-byte loads, the whole group reads 256 contiguous bytes per j) and the matching running sums; the next four cells of the wave are
// requested before the current ones are used.  Every group keeps its own running maximum / sum / weighted latent; groups, then waves, are merged at the
// end together with the sink term.  NJ = ceil((kv_rank + rot) / 64); VEC: rows are 16-byte aligned (kv_rank + rot a multiple of 4).
template <int NJ, bool VEC>
__global__ __launch_bounds__(512) void latent_attn_kernel(LatentAttnArgs a) {
    extern __shared__ float lds[];
    const int KR = a.kv_rank, R = a.rot, L = KR + R, LP = NJ * 64;
    const int NW = blockDim.x >> 6;
    float *qv = lds;                                            // [LP] (zero beyond L)
    float *wm = lds + LP, *wl = wm + NW, *wacc = wl + NW;        // [NW], [NW], [NW][LP]
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 4, li = lane & 15;
    const int tpos = a.tok_pos[t];
    const uint64_t sbit = 1ull << (a.tok_seq[t] & 63);
    for (int i = tid; i < LP; i += blockDim.x) {
        float v = 0.0f;
        if (i < KR) v = a.qa[(size_t)t * a.ld_qa + (size_t)h * KR + i];
        else if (i < L) {
            const float *qr = a.q + (size_t)t * a.ld_q + (size_t)h * (a.dim + R) + a.dim;
            const int r = i - KR;
            if (r < a.rot_dims) {
                const int pr = r >> 1;
                const float ang = (float)tpos * a.rot_freq[pr], c = cosf(ang) * a.rot_mscale, sn = sinf(ang) * a.rot_mscale;
                const float u = qr[2 * pr], w = qr[2 * pr + 1];
                v = (r & 1) ? w * c + u * sn : u * c - w * sn;
            } else v = qr[r];
        }
        qv[i] = v;
    }
    __syncthreads();
    float acc[NJ][4], cur[NJ][4], nxt[NJ][4];
#pragma unroll
    for (int j = 0; j < NJ; j++)
#pragma unroll
        for (int e = 0; e < 4; e++) { acc[j][e] = 0.0f; cur[j][e] = 0.0f; nxt[j][e] = 0.0f; }
    float m = -INFINITY, l = 0.0f;
    int n_kv = *a.n_kv_dev;
    if (a.tok_hi) n_kv = a.tok_hi[t] < n_kv ? a.tok_hi[t] : n_kv;
    const int stride = NW * 4;
    // gridDim.z > 1 (single-token steps): the scanned range is cut into that many runs of cells, one workgroup each; the runs' records are merged by
    // latent_attn_merge_kernel
    int c_lo = 0, c_hi = n_kv;
    if (gridDim.z > 1) {
        const int per = ((n_kv + (int)gridDim.z - 1) / (int)gridDim.z + stride - 1) / stride * stride;
        c_lo = (int)blockIdx.z * per;
        c_hi = c_lo + per < n_kv ? c_lo + per : n_kv;
    }
    const auto visible = [&](int c) {
        if (c >= c_hi) return false;
        const int cp = a.cell_pos[c];
        return cp >= 0 && cp <= tpos && (a.cell_seq[c] & sbit) != 0 && !(a.window > 0 && tpos - cp >= a.window);
    };
    const auto fetch = [&](int c, bool vis, float (&dst)[NJ][4]) {
        const float *row = a.cache + (size_t)c * L;
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const int e0 = 64 * j + 4 * li;
            if (VEC) {
                float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                if (vis && e0 < L) v = *reinterpret_cast<const float4 *>(row + e0);
                dst[j][0] = v.x; dst[j][1] = v.y; dst[j][2] = v.z; dst[j][3] = v.w;
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) dst[j][e] = vis && e0 + e < L ? row[e0 + e] : 0.0f;
            }
        }
    };
    int c = c_lo + wave * 4 + g;
    bool vis = visible(c);
    fetch(c, vis, cur);
    for (int c0 = c_lo; c0 < c_hi; c0 += stride) {              // (uniform trip count: the shuffles below are executed by whole waves)
        const int cn = c + stride;
        const bool visn = visible(cn);
        fetch(cn, visn, nxt);
        float dot = 0.0f;
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const float4 q4 = *reinterpret_cast<const float4 *>(qv + 64 * j + 4 * li);
            dot = fmaf(cur[j][0], q4.x, dot); dot = fmaf(cur[j][1], q4.y, dot); dot = fmaf(cur[j][2], q4.z, dot); dot = fmaf(cur[j][3], q4.w, dot);
        }
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) dot += __shfl_xor(dot, o, 64);
        if (vis) {
            const float sc = dot * a.scale;
            const float mn = fmaxf(m, sc), alpha = expf(m - mn), p = expf(sc - mn);   // (m = -inf at the group's first cell: alpha = 0)
            l = l * alpha + p;
#pragma unroll
            for (int j = 0; j < NJ; j++)
#pragma unroll
                for (int e = 0; e < 4; e++) acc[j][e] = acc[j][e] * alpha + p * cur[j][e];
            m = mn;
        }
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) cur[j][e] = nxt[j][e];
        c = cn; vis = visn;
    }
    // the four groups of a wave -> one record per wave
    float M = fmaxf(m, __shfl_xor(m, 16, 64));
    M = fmaxf(M, __shfl_xor(M, 32, 64));
    const float sg = l > 0.0f ? expf(m - M) : 0.0f;
    l *= sg;
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
#pragma unroll
    for (int j = 0; j < NJ; j++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
            float v = acc[j][e] * sg;
            v += __shfl_xor(v, 16, 64);
            v += __shfl_xor(v, 32, 64);
            if (g == 0) wacc[wave * LP + 64 * j + 4 * li + e] = v;
        }
    if (lane == 0) { wm[wave] = M; wl[wave] = l; }
    __syncthreads();
    if (gridDim.z > 1) {                                        // this run's record: maximum, sum, weighted latent (no sink: the merge adds it once)
        float *rec = a.part + (((size_t)t * a.H + h) * gridDim.z + blockIdx.z) * (size_t)(KR + 2);
        float Ms = -INFINITY;
        for (int w = 0; w < NW; w++) if (wl[w] > 0.0f) Ms = fmaxf(Ms, wm[w]);
        float ls = 0.0f;
        for (int w = 0; w < NW; w++) ls += wl[w] > 0.0f ? wl[w] * expf(wm[w] - Ms) : 0.0f;
        if (tid == 0) { rec[0] = Ms; rec[1] = ls; }
        for (int i = tid; i < KR; i += blockDim.x) {
            float o = 0.0f;
            for (int w = 0; w < NW; w++) o += wl[w] > 0.0f ? wacc[w * LP + i] * expf(wm[w] - Ms) : 0.0f;
            rec[2 + i] = o;
        }
        return;
    }
    float MM = a.sink ? a.sink[h] : -INFINITY;
    for (int w = 0; w < NW; w++) MM = fmaxf(MM, wm[w]);
    float den = a.sink ? expf(a.sink[h] - MM) : 0.0f;
    for (int w = 0; w < NW; w++) den += wl[w] > 0.0f ? wl[w] * expf(wm[w] - MM) : 0.0f;
    const float inv = den > 0.0f ? 1.0f / den : 0.0f;
    for (int i = tid; i < KR; i += blockDim.x) {
        float o = 0.0f;
        for (int w = 0; w < NW; w++) o += wl[w] > 0.0f ? wacc[w * LP + i] * expf(wm[w] - MM) : 0.0f;
        a.out[(size_t)t * a.ld_out + (size_t)h * KR + i] = o * inv;
    }
}

__global__ __launch_bounds__(256) void latent_attn_merge_kernel(LatentAttnArgs a, int splits) {
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, KR = a.kv_rank;
    const float *rec = a.part + ((size_t)t * a.H + h) * splits * (size_t)(KR + 2);
    float MM = a.sink ? a.sink[h] : -INFINITY;
    for (int s = 0; s < splits; s++) if (rec[(size_t)s * (KR + 2) + 1] > 0.0f) MM = fmaxf(MM, rec[(size_t)s * (KR + 2)]);
    float den = a.sink ? expf(a.sink[h] - MM) : 0.0f;
    for (int s = 0; s < splits; s++) { const float *r = rec + (size_t)s * (KR + 2); den += r[1] > 0.0f ? r[1] * expf(r[0] - MM) : 0.0f; }
    const float inv = den > 0.0f ? 1.0f / den : 0.0f;
    for (int i = tid; i < KR; i += 256) {
        float o = 0.0f;
        for (int s = 0; s < splits; s++) { const float *r = rec + (size_t)s * (KR + 2); o += r[1] > 0.0f ? r[2 + i] * expf(r[0] - MM) : 0.0f; }
        a.out[(size_t)t * a.ld_out + (size_t)h * KR + i] = o * inv;
    }
}

template <int NJ>
static hipError_t launch_latent_attn_nj(const LatentAttnArgs &a, hipStream_t st) {
    // few (token, head) pairs - single-token steps - get eight waves each: more cells in flight where the grid alone cannot fill the device
    const int nw = (long long)a.T * a.H <= 1024 ? 8 : 4;
    const size_t lds = (size_t)(NJ * 64 + 2 * nw + nw * NJ * 64) * sizeof(float);
    const bool vec = ((a.kv_rank + a.rot) & 3) == 0 && (reinterpret_cast<uintptr_t>(a.cache) & 15) == 0;
    const int splits = a.part && a.splits > 1 ? a.splits : 1;
    const dim3 grid((unsigned)a.T, (unsigned)a.H, (unsigned)splits);
    if (vec) hipLaunchKernelGGL((latent_attn_kernel<NJ, true>), grid, dim3(64 * nw), lds, st, a);
    else hipLaunchKernelGGL((latent_attn_kernel<NJ, false>), grid, dim3(64 * nw), lds, st, a);
    if (splits > 1) hipLaunchKernelGGL(latent_attn_merge_kernel, dim3((unsigned)a.T, (unsigned)a.H), dim3(256), 0, st, a, splits);
    return hipGetLastError();
}

}  // namespace

bool latent_attn_shape_ok(int kv_rank, int rot) { return kv_rank >= 1 && rot >= 0 && kv_rank + rot <= LA_MAX_L; }

hipError_t launch_latent_prep(const LatentPrepArgs &a, hipStream_t st) {
    if (a.T <= 0) return hipSuccess;
    if (a.rot_dims > a.rot || (a.rot_dims & 1)) return hipErrorInvalidValue;
    hipLaunchKernelGGL(latent_prep_kernel, dim3((unsigned)a.T), dim3(256), 0, st, a);
    return hipGetLastError();
}

hipError_t launch_latent_attn(const LatentAttnArgs &a, hipStream_t st) {
    if (a.T <= 0) return hipSuccess;
    if (!latent_attn_shape_ok(a.kv_rank, a.rot) || a.rot_dims > a.rot || (a.rot_dims & 1)) return hipErrorInvalidValue;
    const int L = a.kv_rank + a.rot;
    if (L <= 128) return launch_latent_attn_nj<2>(a, st);
    if (L <= 320) return launch_latent_attn_nj<5>(a, st);
    if (L <= 576) return launch_latent_attn_nj<9>(a, st);
    return launch_latent_attn_nj<17>(a, st);
}

}  // namespace mi355
