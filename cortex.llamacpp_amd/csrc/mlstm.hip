// mlstm.hip — the matrix-memory recurrence (mLSTM of the xLSTM family), token by token with the state in registers.
//
// Per head: a state matrix S [dim][vdim], a normaliser n [dim] and a running maximum m of the log gates, all f32, one set per sequence slot.  For a token
// with query q (already scaled by dim^-1/2 here), key k, value v and the pre-activations of the two gates:
//     i = cap tanh(i_pre / cap)            f = logsigmoid(cap tanh(f_pre / cap))        (both made for the whole batch at once: launch_mlstm_gates)
//     m' = max(f + m, i)     S' = e^(f + m - m') S + e^(i - m') k v^T     n' likewise with k alone
//     o  = S'^T q / (max(|n' . q|, e^(-m')) + 1e-6)
// A state that has seen nothing is S = 0, n = 0, m = 0.  The columns of S evolve independently given the gates, so a workgroup owns 64 columns of one head of
// one sequence segment: lane = column, the four waves split the dim rows (each thread keeps its rows of its column - and of n - in registers), the per-token
// partial sums of S^T q and n . q cross the waves through LDS.  A segment is a run of consecutive rows of the batch that belong to one sequence: a prompt,
// a portion of one, or a single decoded token - the same code, started from the slot's state and ending with the state written back.
// mlstm_out: per head, the output divided by its root mean square, times the mixer's norm weight, times sigmoid of the output gate's pre-activation.
#include "kernels.h"

namespace mi355 {

namespace {

template <int DPER>
__global__ __launch_bounds__(256) void mlstm_scan_kernel(MlstmArgs a) {
    __shared__ float sq[4 * DPER], sk[4 * DPER], red[4][64], redn[4];
    const int seg = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, j = tid & 63, dg = tid >> 6;
    const int col = blockIdx.z * 64 + j, d0 = dg * DPER;
    const int H = a.H, D = a.D, VD = a.VD;
    const int start = a.seg_start[seg], len = a.seg_len[seg], slot = a.seg_slot[seg];
    float *Sg = a.S + ((size_t)slot * H + h) * (size_t)D * VD;
    float *ng = a.n + ((size_t)slot * H + h) * D;
    float *mg = a.m + (size_t)slot * H + h;
    float S[DPER], n[DPER];
#pragma unroll
    for (int e = 0; e < DPER; e++) {
        const int d = d0 + e;
        S[e] = d < D && col < VD ? Sg[(size_t)d * VD + col] : 0.0f;
        n[e] = d < D ? ng[d] : 0.0f;
    }
    float m = *mg;
    const float qscale = 1.0f / sqrtf((float)D);
    const int off_k = H * D, off_v = 2 * H * D, off_i = 2 * H * D + 2 * H * VD, off_f = off_i + H;
    // the next token's inputs are requested while the current one is being used (a request per token in the dependency chain would cost a memory
    // round trip each); the gate columns already hold the log gates (mlstm_gates_kernel)
    constexpr int NLD = (4 * DPER + 255) / 256;
    float rq[NLD], rk[NLD], rv, rig, rfg;
    const auto request = [&](int t) {
        const float *row = a.p + (size_t)(start + t) * a.ld_p;
#pragma unroll
        for (int u = 0; u < NLD; u++) {
            const int d = tid + 256 * u;
            rq[u] = d < D ? row[h * D + d] : 0.0f;
            rk[u] = d < D ? row[off_k + h * D + d] : 0.0f;
        }
        rv = col < VD ? row[off_v + h * VD + col] : 0.0f;
        rig = row[off_i + h];
        rfg = row[off_f + h];
    };
    if (len > 0) request(0);
    for (int t = 0; t < len; t++) {
        __syncthreads();                                        // (the previous token's partial sums and q / k rows have been read)
#pragma unroll
        for (int u = 0; u < NLD; u++) {
            const int d = tid + 256 * u;
            if (d < 4 * DPER) { sq[d] = rq[u] * qscale; sk[d] = rk[u]; }
        }
        const float v = rv, ig = rig, fg = rfg;
        if (t + 1 < len) request(t + 1);
        const float mn = fmaxf(fg + m, ig), ea = expf(fg + m - mn), eb = expf(ig - mn);
        m = mn;
        __syncthreads();
        float num = 0.0f, nq = 0.0f;
#pragma unroll
        for (int e = 0; e < DPER; e++) {
            const float kd = eb * sk[d0 + e], q = sq[d0 + e];
            S[e] = fmaf(ea, S[e], kd * v);
            n[e] = fmaf(ea, n[e], kd);
            num = fmaf(S[e], q, num);
            nq = fmaf(n[e], q, nq);
        }
        red[dg][j] = num;
        if (j == 0) redn[dg] = nq;
        __syncthreads();
        if (dg == 0 && col < VD) {
            const float nt = (red[0][j] + red[1][j]) + (red[2][j] + red[3][j]);
            const float qt = (redn[0] + redn[1]) + (redn[2] + redn[3]);
            a.o[(size_t)(start + t) * a.ld_o + (size_t)h * VD + col] = nt / (fmaxf(fabsf(qt), expf(-m)) + 1e-6f);
        }
    }
#pragma unroll
    for (int e = 0; e < DPER; e++) {
        const int d = d0 + e;
        if (d < D && col < VD) Sg[(size_t)d * VD + col] = S[e];
        if (d < D && blockIdx.z == 0 && j == 0) ng[d] = n[e];
    }
    if (blockIdx.z == 0 && tid == 0) *mg = m;
}

// the two log gates of every (token, head), in place over their pre-activations: i = cap tanh((x + b_i) / cap), f = logsigmoid(cap tanh((x + b_f) / cap))
__global__ void mlstm_gates_kernel(float *p, int ld_p, int off_i, int H, int T, const float *ib, const float *fb, float cap) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= T * H) return;
    const int t = i / H, h = i - t * H;
    float *row = p + (size_t)t * ld_p + off_i;
    const float ig = cap * tanhf((row[h] + (ib ? ib[h] : 0.0f)) / cap);
    const float fz = cap * tanhf((row[H + h] + (fb ? fb[h] : 0.0f)) / cap);
    row[h] = ig;
    row[H + h] = fminf(fz, 0.0f) - log1pf(expf(-fabsf(fz)));
}

__global__ __launch_bounds__(64) void mlstm_out_kernel(const float *o, int ld_o, const float *p, int ld_p, int off_g, const float *w, int H, int VD, float eps,
                                                       float *y, int ld_y) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float *orow = o + (size_t)t * ld_o + (size_t)h * VD;
    float ss = 0.0f;
    for (int i = lane; i < VD; i += 64) { const float v = orow[i]; ss = fmaf(v, v, ss); }
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) ss += __shfl_xor(ss, s, 64);
    const float inv = 1.0f / sqrtf(ss / (float)VD + eps);
    for (int i = lane; i < VD; i += 64) {
        const float g = p[(size_t)t * ld_p + off_g + h * VD + i];
        y[(size_t)t * ld_y + (size_t)h * VD + i] = orow[i] * inv * w[h * VD + i] * (1.0f / (1.0f + expf(-g)));
    }
}

__global__ void mlstm_state_reset_kernel(float *S, size_t n_s, float *n, size_t n_n, float *m, size_t n_m) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n_s) S[i] = 0.0f;
    if (i < n_n) n[i] = 0.0f;
    if (i < n_m) m[i] = 0.0f;
}

}  // namespace

bool mlstm_shape_ok(int D, int VD) { return D >= 1 && D <= 512 && VD >= 1; }

hipError_t launch_mlstm_gates(const MlstmArgs &a, int T, hipStream_t st) {
    if (T <= 0) return hipSuccess;
    hipLaunchKernelGGL(mlstm_gates_kernel, dim3((unsigned)((T * a.H + 255) / 256)), dim3(256), 0, st, const_cast<float *>(a.p), a.ld_p,
                       2 * a.H * a.D + 2 * a.H * a.VD, a.H, T, a.i_bias, a.f_bias, a.gate_cap);
    return hipGetLastError();
}

hipError_t launch_mlstm_scan(const MlstmArgs &a, hipStream_t st) {
    if (a.n_seg <= 0) return hipSuccess;
    if (!mlstm_shape_ok(a.D, a.VD)) return hipErrorInvalidValue;
    const dim3 grid((unsigned)a.n_seg, (unsigned)a.H, (unsigned)((a.VD + 63) / 64));
    if (a.D <= 32) hipLaunchKernelGGL(mlstm_scan_kernel<8>, grid, dim3(256), 0, st, a);
    else if (a.D <= 64) hipLaunchKernelGGL(mlstm_scan_kernel<16>, grid, dim3(256), 0, st, a);
    else if (a.D <= 128) hipLaunchKernelGGL(mlstm_scan_kernel<32>, grid, dim3(256), 0, st, a);
    else if (a.D <= 256) hipLaunchKernelGGL(mlstm_scan_kernel<64>, grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL(mlstm_scan_kernel<128>, grid, dim3(256), 0, st, a);
    return hipGetLastError();
}

hipError_t launch_mlstm_out(const float *o, int ld_o, const float *p, int ld_p, int off_g, const float *w, int T, int H, int VD, float eps, float *y, int ld_y,
                            hipStream_t st) {
    if (T <= 0) return hipSuccess;
    hipLaunchKernelGGL(mlstm_out_kernel, dim3((unsigned)T, (unsigned)H), dim3(64), 0, st, o, ld_o, p, ld_p, off_g, w, H, VD, eps, y, ld_y);
    return hipGetLastError();
}

hipError_t launch_mlstm_state_reset(float *S, size_t n_s, float *n, size_t n_n, float *m, size_t n_m, hipStream_t st) {
    const size_t mx = n_s > n_n ? (n_s > n_m ? n_s : n_m) : (n_n > n_m ? n_n : n_m);
    if (!mx) return hipSuccess;
    hipLaunchKernelGGL(mlstm_state_reset_kernel, dim3((unsigned)((mx + 255) / 256)), dim3(256), 0, st, S, n_s, n, n_n, m, n_m);
    return hipGetLastError();
}

}  // namespace mi355
