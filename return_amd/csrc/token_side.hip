// Per-layer token input: a second, narrow embedding of the token, gated by the residual stream,
// projected up and added to the stream through an RMS norm of its own. For row t with token id:
//     h_t += delta_t                              (the pending output of the part before, if any)
//     a[r] = sum_c gate[r][c] * h_t[c]            r < S
//     g[r] = gelu_tanh(a[r]) * table[id][off + r]
//     y[c] = sum_r proj[c][r] * g[r]
//     h_t[c] += y[c] / sqrt(mean_c y[c]^2 + eps) * w[c]
// gelu_tanh(x) = 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))). Sums, the norm and the stream are
// 32-bit; gate [S, H], proj [H, S] and the table [vocab, ld_table] are in the storage type.
// One workgroup per row: every thread sums its columns' share of the gate products (SB of them a pass), the
// shares are added over the workgroup through LDS, then every thread forms its columns of y.
#include "common.h"

#define TS_MAX_S 512
#define TS_THREADS 256
#define TS_MAX_CPT 32        // columns per thread: H <= 256 * 32

template <typename T, int SB>
__global__ __launch_bounds__(TS_THREADS) void token_side_kernel(
    float* __restrict__ h, const T* __restrict__ delta, const int* __restrict__ ids, const T* __restrict__ table,
    long long ld_table, int off, const T* __restrict__ gate, const T* __restrict__ proj, const float* __restrict__ w,
    float eps, int H, int S) {
    __shared__ float part[TS_THREADS / 64][SB];
    __shared__ float g_s[TS_MAX_S];
    __shared__ float red[16];
    const int t = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float* hr = h + (size_t)t * H;
    for (int r0 = 0; r0 < S; r0 += SB) {                 // SB gate rows a pass; the first pass adds delta into the stream
        float a[SB];
#pragma unroll
        for (int r = 0; r < SB; ++r) a[r] = 0.f;
        for (int c = tid; c < H; c += TS_THREADS) {
            float v = hr[c];
            if (r0 == 0 && delta != nullptr) {
                v += to_f(delta[(size_t)t * H + c]);
                hr[c] = v;                               // (read again by this thread only)
            }
#pragma unroll
            for (int r = 0; r < SB; ++r)
                if (r0 + r < S) a[r] = fmaf(to_f(gate[(size_t)(r0 + r) * H + c]), v, a[r]);
        }
#pragma unroll
        for (int r = 0; r < SB; ++r) {
            const float v = wave_sum(a[r]);
            if (lane == 0) part[wave][r] = v;
        }
        __syncthreads();
        if (tid < SB && r0 + tid < S) {
            float x = 0.f;
            for (int wv = 0; wv < TS_THREADS / 64; ++wv) x += part[wv][tid];
            const float inner = 0.7978845608028654f * (x + 0.044715f * x * x * x);
            const float e = to_f(table[(size_t)ids[t] * ld_table + off + r0 + tid]);
            g_s[r0 + tid] = 0.5f * x * (1.f + tanhf(inner)) * e;
        }
        __syncthreads();
    }
    float y[TS_MAX_CPT];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < TS_MAX_CPT; ++i) {
        const int c = tid + i * TS_THREADS;
        y[i] = 0.f;
        if (c < H) {
            float v = 0.f;
            for (int r = 0; r < S; ++r) v = fmaf(to_f(proj[(size_t)c * S + r]), g_s[r], v);
            y[i] = v;
            ss = fmaf(v, v, ss);
        }
    }
    ss = block_sum(ss, red);
    const float rstd = 1.0f / sqrtf(ss / (float)H + eps);
#pragma unroll
    for (int i = 0; i < TS_MAX_CPT; ++i) {
        const int c = tid + i * TS_THREADS;
        if (c < H) hr[c] += y[i] * rstd * w[c];
    }
}

extern "C" int ra_token_side(float* h, const void* delta, const int* ids, const void* table, long long ld_table, int off,
                             const void* gate, const void* proj, const float* w, float eps, int T_tokens, int H, int S,
                             int dtype, void* stream) {
    if (T_tokens <= 0) return RA_OK;
    if (S < 1 || S > TS_MAX_S || H < 1 || H > TS_THREADS * TS_MAX_CPT || off < 0 || ld_table < off + S) return RA_ERR_ARG;
    dim3 grid(T_tokens), block(TS_THREADS);
    hipStream_t st = (hipStream_t)stream;
#define TS_GO(T_, SB_)                                                                                         \
    hipLaunchKernelGGL((token_side_kernel<T_, SB_>), grid, block, 0, st, h, (const T_*)delta, ids, (const T_*)table, \
                       ld_table, off, (const T_*)gate, (const T_*)proj, w, eps, H, S)
    if (dtype == RA_DTYPE_F32) {
        if (S <= 16) TS_GO(float, 16); else if (S <= 32) TS_GO(float, 32); else TS_GO(float, 64);
    } else if (dtype == RA_DTYPE_BF16) {
        if (S <= 16) TS_GO(bf16, 16); else if (S <= 32) TS_GO(bf16, 32); else TS_GO(bf16, 64);
    } else {
        return RA_ERR_ARG;
    }
#undef TS_GO
    return ra_launch_status();
}
