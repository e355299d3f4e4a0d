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

// The same for bfloat16 with 16-byte loads (H % 8 == 0, S % 8 == 0, S <= TS_MAX_S), R rows of the stream
// a workgroup: the rows (with delta added) sit in LDS in 32-bit; a wave takes every fourth gate row and
// forms its product with all R stream rows, each lane eight columns at a time, so that all of a row's
// loads are on their way at once and a gate row is read once for R rows; then a thread forms its columns of
// y for all R rows from one read of the projection's row.
template <int R, int NTH>
__global__ __launch_bounds__(NTH) void token_side_bf16x8_kernel(
    float* __restrict__ h, const bf16* __restrict__ delta, const int* __restrict__ ids, const bf16* __restrict__ table,
    long long ld_table, int off, const bf16* __restrict__ gate, const bf16* __restrict__ proj,
    const float* __restrict__ w, float eps, int T_tokens, int H, int S) {
    extern __shared__ __attribute__((aligned(16))) float ts_smem[];
    float* x_s = ts_smem;                        // [R][H]
    float* g_s = x_s + (size_t)R * H;            // [R][S]
    float* red = g_s + R * S;                    // [R][waves]
    const int t0 = blockIdx.x * R, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int rows = min(R, T_tokens - t0);
    for (int idx = tid * 4; idx < R * H; idx += NTH * 4) {
        const int rr = idx / H, c = idx - rr * H;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (rr < rows) {
            v = *reinterpret_cast<const float4*>(h + (size_t)(t0 + rr) * H + c);
            if (delta != nullptr) {
                const uint2 d = *reinterpret_cast<const uint2*>(delta + (size_t)(t0 + rr) * H + c);
                v.x += __uint_as_float(d.x << 16); v.y += __uint_as_float(d.x & 0xffff0000u);
                v.z += __uint_as_float(d.y << 16); v.w += __uint_as_float(d.y & 0xffff0000u);
            }
        }
        *reinterpret_cast<float4*>(x_s + idx) = v;
    }
    __syncthreads();
    for (int r = wave; r < S; r += (NTH / 64)) {
        float a[R];
#pragma unroll
        for (int rr = 0; rr < R; ++rr) a[rr] = 0.f;
        for (int c = lane * 8; c < H; c += 512) {
            const uint4 gw = *reinterpret_cast<const uint4*>(gate + (size_t)r * H + c);
            const float g8[8] = {__uint_as_float(gw.x << 16), __uint_as_float(gw.x & 0xffff0000u),
                                 __uint_as_float(gw.y << 16), __uint_as_float(gw.y & 0xffff0000u),
                                 __uint_as_float(gw.z << 16), __uint_as_float(gw.z & 0xffff0000u),
                                 __uint_as_float(gw.w << 16), __uint_as_float(gw.w & 0xffff0000u)};
#pragma unroll
            for (int rr = 0; rr < R; ++rr) {
                const float4 x0 = *reinterpret_cast<const float4*>(x_s + (size_t)rr * H + c);
                const float4 x1 = *reinterpret_cast<const float4*>(x_s + (size_t)rr * H + c + 4);
                a[rr] = fmaf(g8[0], x0.x, a[rr]); a[rr] = fmaf(g8[1], x0.y, a[rr]);
                a[rr] = fmaf(g8[2], x0.z, a[rr]); a[rr] = fmaf(g8[3], x0.w, a[rr]);
                a[rr] = fmaf(g8[4], x1.x, a[rr]); a[rr] = fmaf(g8[5], x1.y, a[rr]);
                a[rr] = fmaf(g8[6], x1.z, a[rr]); a[rr] = fmaf(g8[7], x1.w, a[rr]);
            }
        }
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            const float x = wave_sum(a[rr]);
            if (lane == 0 && rr < rows) {
                const float inner = 0.7978845608028654f * (x + 0.044715f * x * x * x);
                const float e = to_f(table[(size_t)ids[t0 + rr] * ld_table + off + r]);
                g_s[rr * S + r] = 0.5f * x * (1.f + tanhf(inner)) * e;
            }
        }
    }
    __syncthreads();
    float y[R][(4096 / NTH)];                  // H <= 4096 in this form
    float ss[R];
#pragma unroll
    for (int rr = 0; rr < R; ++rr) ss[rr] = 0.f;
#pragma unroll
    for (int i = 0; i < (4096 / NTH); ++i) {
        const int c = tid + i * NTH;
#pragma unroll
        for (int rr = 0; rr < R; ++rr) y[rr][i] = 0.f;
        if (c < H) {
            for (int r8 = 0; r8 < S; r8 += 8) {
                const uint4 pw = *reinterpret_cast<const uint4*>(proj + (size_t)c * S + r8);
                const float p8[8] = {__uint_as_float(pw.x << 16), __uint_as_float(pw.x & 0xffff0000u),
                                     __uint_as_float(pw.y << 16), __uint_as_float(pw.y & 0xffff0000u),
                                     __uint_as_float(pw.z << 16), __uint_as_float(pw.z & 0xffff0000u),
                                     __uint_as_float(pw.w << 16), __uint_as_float(pw.w & 0xffff0000u)};
#pragma unroll
                for (int rr = 0; rr < R; ++rr)
#pragma unroll
                    for (int k = 0; k < 8; ++k) y[rr][i] = fmaf(p8[k], g_s[rr * S + r8 + k], y[rr][i]);
            }
#pragma unroll
            for (int rr = 0; rr < R; ++rr) ss[rr] = fmaf(y[rr][i], y[rr][i], ss[rr]);
        }
    }
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
        const float v = wave_sum(ss[rr]);
        if (lane == 0) red[rr * (NTH / 64) + wave] = v;
    }
    __syncthreads();
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
        if (rr >= rows) break;
        float tot = 0.f;
        for (int wv = 0; wv < NTH / 64; ++wv) tot += red[rr * (NTH / 64) + wv];      // (the same order in every thread)
        const float rstd = 1.0f / sqrtf(tot / (float)H + eps);
#pragma unroll
        for (int i = 0; i < (4096 / NTH); ++i) {
            const int c = tid + i * NTH;
            if (c < H) h[(size_t)(t0 + rr) * H + c] = x_s[(size_t)rr * H + c] + y[rr][i] * rstd * w[c];
        }
    }
}

template <int R, int NTH>
static int token_side_x8_launch(hipStream_t st, float* h, const void* delta, const int* ids, const void* table,
                                long long ld_table, int off, const void* gate, const void* proj, const float* w, float eps,
                                int T_tokens, int H, int S) {
    const size_t lds = sizeof(float) * ((size_t)R * H + (size_t)R * S + R * (NTH / 64));
    if (lds > 64 * 1024 &&
        hipFuncSetAttribute((const void*)token_side_bf16x8_kernel<R, NTH>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess)
        return RA_ERR_LAUNCH;
    hipLaunchKernelGGL((token_side_bf16x8_kernel<R, NTH>), dim3((T_tokens + R - 1) / R), dim3(NTH), lds, st, h,
                       (const bf16*)delta, ids, (const bf16*)table, ld_table, off, (const bf16*)gate, (const bf16*)proj, w,
                       eps, T_tokens, H, S);
    return ra_launch_status();
}

extern "C" int ra_token_side(float* h, const void* delta, const int* ids, const void* table, long long ld_table, int off,
                             const void* gate, const void* proj, const float* w, float eps, int T_tokens, int H, int S,
                             int dtype, void* stream) {
    if (T_tokens <= 0) return RA_OK;
    if (S < 1 || S > TS_MAX_S || H < 1 || H > TS_THREADS * TS_MAX_CPT || off < 0 || ld_table < off + S) return RA_ERR_ARG;
    dim3 grid(T_tokens), block(TS_THREADS);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == RA_DTYPE_BF16 && H % 8 == 0 && S % 8 == 0 && H <= 4096) {
        // many rows: four a workgroup, so that the two matrices are read once for four rows
        if (T_tokens >= 256)
            return token_side_x8_launch<4, 256>(st, h, delta, ids, table, ld_table, off, gate, proj, w, eps, T_tokens, H, S);
        // few rows: sixteen waves a row, so that a row's loads are spread over four times the threads
        if (T_tokens <= 64)
            return token_side_x8_launch<1, 1024>(st, h, delta, ids, table, ld_table, off, gate, proj, w, eps, T_tokens, H, S);
        return token_side_x8_launch<1, 256>(st, h, delta, ids, table, ld_table, off, gate, proj, w, eps, T_tokens, H, S);
    }
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
