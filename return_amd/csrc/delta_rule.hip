// Gated delta rule with one decay per key channel, as one kernel over the rows of a step.
//
// Per head, with S [D, V] in 32-bit carried from token to token for each request:
//     S <- diag(g_t) S;   u = beta_t (v_t - S^T k_t);   S <- S + k_t u^T;   o_t = S^T q_t
// (the read-out sees the token's own write). Around it, all in 32-bit:
//     q_t, k_t: unit vectors per head, x / sqrt(sum x^2 + 1e-6), q times D^-1/2
//     beta_t = sigmoid(b_t)
//     g_t[i] = exp(-exp(A_log[h]) * softplus(dt_bias[h,i] + sum_r a1_t[r] * Wa2[h,i,r]))
//     out_t[j] = o_t[j] / sqrt(mean_j o_t[j]^2 + eps) * norm_w[j] * sigmoid(sum_r g1_t[r] * Wg2[h,j,r])
// Inputs: qkv, the rows after the short convolution and its activation, [q heads | k heads | v heads]
// (G heads of D for q and k, H heads of V for v; head h reads q/k head h / (H/G)); z, the rows of the
// fused input projection, of which beta (H columns at off_b), a1 (ra columns at off_a) and g1 (rg
// columns at off_g) are read; the second factors of the two low-rank maps transposed, fp32
// [ra, H*D] and [rg, H*V].
//
// A workgroup takes one (head, request) and walks the request's rows in chunks of DR_TC: first
// everything that does not depend on S is prepared for the chunk in LDS by all threads (the decay's
// low-rank map, whose second factor's rows for this head are copied into LDS once when they fit,
// softplus, exponentials, the unit vectors), then the recurrence runs over the chunk
// without a barrier, then the chunk's read-outs are normed, gated and stored. In the recurrence a
// column j of S belongs to RS neighbouring lanes, each with DPT rows in registers; the two sums
// over rows are finished by lane swaps.
#include "common.h"

#define DR_TC 16
#define DR_PAD 4

__device__ __forceinline__ float dr_sigmoid(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float dr_softplus(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// Sum over the RS (1, 2, 4 or 8) neighbouring lanes that share a column, in every one of them, by
// data-parallel moves inside a row of 16 lanes: partner lane ^ 1, then lane ^ 2, then the other quad
// of the eight (mirrored: after the first two steps a quad's lanes all hold the quad's sum).
__device__ __forceinline__ float dr_group_sum(float v, int RS) {
    if (RS >= 2)
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    if (RS >= 4)
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    if (RS >= 8)
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
    return v;
}

template <typename T, int DPT>
__global__ __launch_bounds__(512) void delta_rule_kernel(
    const T* __restrict__ qkv, long long ld_qkv, const T* __restrict__ z, long long ld_z, int off_b, int off_a,
    int ra, int off_g, int rg, const float* __restrict__ w_a2t, const float* __restrict__ w_g2t,
    const float* __restrict__ A_log, const float* __restrict__ dt_bias, const float* __restrict__ norm_w,
    float eps, float* __restrict__ S, const int* __restrict__ cu_q, const int* __restrict__ slot_ids,
    T* __restrict__ out, int H, int G, int D, int V, int RS, int staged) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int tid = threadIdx.x, NT = blockDim.x, lane = tid & 63, wave = tid >> 6, n_waves = NT >> 6;
    const int h = blockIdx.x, s = blockIdx.y, kvh = h / (H / G);
    const int base = cu_q[s], q_len = cu_q[s + 1] - base;
    if (q_len <= 0) return;
    const int PS = DPT + DR_PAD;                    // a lane group's rows in LDS, padded against bank conflicts
    const int DP = RS * PS;
    const int rap = (ra + 3) & ~3, rgp = (rg + 3) & ~3;   // the ranks as rows of whole float4 (zeros beyond)
    float* k_s = smem;                              // [TC][DP]
    float* q_s = k_s + DR_TC * DP;                  // [TC][DP]
    float* g_s = q_s + DR_TC * DP;                  // [TC][DP]
    float* v_s = g_s + DR_TC * DP;                  // [TC][V]
    float* o_s = v_s + DR_TC * V;                   // [TC][V]
    float* a1_s = o_s + DR_TC * V;                  // [TC][rap]
    float* g1_s = a1_s + DR_TC * rap;               // [TC][rgp]
    float* beta_s = g1_s + DR_TC * rgp;             // [TC]
    float* rstd_s = beta_s + DR_TC;                 // [TC]
    // staged: this head's rows of the two low-rank second factors sit in LDS for the whole walk
    float* wa_s = rstd_s + DR_TC;                   // [rap][D]
    float* wg_s = wa_s + (staged ? rap * D : 0);    // [rgp][V]
    if (staged) {
        for (int idx = tid; idx < rap * D; idx += NT) {
            const int r = idx / D, i = idx - r * D;
            wa_s[idx] = r < ra ? w_a2t[(size_t)r * H * D + h * D + i] : 0.f;
        }
        for (int idx = tid; idx < rgp * V; idx += NT) {
            const int r = idx / V, jj = idx - r * V;
            wg_s[idx] = r < rg ? w_g2t[(size_t)r * H * V + h * V + jj] : 0.f;
        }
    }

    const int j = tid / RS, rp = tid % RS;
    const bool live = j < V;
    float* Sh = S + ((size_t)slot_ids[s] * H + h) * D * V;
    float st[DPT];
#pragma unroll
    for (int ii = 0; ii < DPT; ++ii) {
        const int i = rp * DPT + ii;
        st[ii] = (live && i < D) ? Sh[(size_t)i * V + j] : 0.f;
    }
    const float neg_a = -expf(A_log[h]);
    const float q_scale = 1.0f / sqrtf((float)D);
    const int Dfull = RS * DPT;

    for (int c0 = 0; c0 < q_len; c0 += DR_TC) {
        const int nt = min(DR_TC, q_len - c0);
        // ---- what the chunk's rows bring, into LDS
        for (int idx = tid; idx < nt * rap; idx += NT) {
            const int tt = idx / rap, r = idx - tt * rap;
            a1_s[idx] = r < ra ? to_f(z[(size_t)(base + c0 + tt) * ld_z + off_a + r]) : 0.f;
        }
        for (int idx = tid; idx < nt * rgp; idx += NT) {
            const int tt = idx / rgp, r = idx - tt * rgp;
            g1_s[idx] = r < rg ? to_f(z[(size_t)(base + c0 + tt) * ld_z + off_g + r]) : 0.f;
        }
        if (tid < nt) beta_s[tid] = dr_sigmoid(to_f(z[(size_t)(base + c0 + tid) * ld_z + off_b + h]));
        for (int idx = tid; idx < nt * V; idx += NT) {
            const int tt = idx / V, jj = idx - tt * V;
            v_s[tt * V + jj] = to_f(qkv[(size_t)(base + c0 + tt) * ld_qkv + 2 * G * D + h * V + jj]);
        }
        __syncthreads();
        // a thread takes one key channel of four rows at a time: a row of the factor is read once for the four
        for (int idx = tid; idx < ((nt + 3) >> 2) * Dfull; idx += NT) {
            const int tg = idx / Dfull, i = idx - tg * Dfull;
            float a[4] = {0.f, 0.f, 0.f, 0.f};
            if (i < D) {
                const float* a1 = a1_s + (tg * 4) * rap;          // (rows beyond nt hold older numbers: never used)
#pragma unroll 2
                for (int r = 0; r < rap; r += 4) {
                    float w4[4];
#pragma unroll
                    for (int x = 0; x < 4; ++x)
                        w4[x] = staged ? wa_s[(r + x) * D + i]
                                       : (r + x < ra ? w_a2t[(size_t)(r + x) * H * D + h * D + i] : 0.f);
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const float4 c4 = *reinterpret_cast<const float4*>(a1 + k * rap + r);
                        a[k] = fmaf(c4.x, w4[0], a[k]);
                        a[k] = fmaf(c4.y, w4[1], a[k]);
                        a[k] = fmaf(c4.z, w4[2], a[k]);
                        a[k] = fmaf(c4.w, w4[3], a[k]);
                    }
                }
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int tt = tg * 4 + k;
                if (tt >= nt) break;
                const int at = tt * DP + (i / DPT) * PS + (i % DPT);
                float kk = 0.f, qq = 0.f, gg = 1.f;
                if (i < D) {
                    const T* row = qkv + (size_t)(base + c0 + tt) * ld_qkv;
                    qq = to_f(row[kvh * D + i]);
                    kk = to_f(row[G * D + kvh * D + i]);
                    gg = expf(neg_a * dr_softplus(a[k] + dt_bias[h * D + i]));
                }
                k_s[at] = kk;
                q_s[at] = qq;
                g_s[at] = gg;
            }
        }
        __syncthreads();
        for (int tt = wave; tt < nt; tt += n_waves) {          // unit vectors: a wave per row
            float sk = 0.f, sq = 0.f;
            for (int i = lane; i < D; i += 64) {
                const int at = tt * DP + (i / DPT) * PS + (i % DPT);
                sk = fmaf(k_s[at], k_s[at], sk);
                sq = fmaf(q_s[at], q_s[at], sq);
            }
            sk = 1.0f / sqrtf(wave_sum(sk) + 1e-6f);
            sq = q_scale / sqrtf(wave_sum(sq) + 1e-6f);
            for (int i = lane; i < D; i += 64) {
                const int at = tt * DP + (i / DPT) * PS + (i % DPT);
                k_s[at] *= sk;
                q_s[at] *= sq;
            }
        }
        __syncthreads();
        // ---- the recurrence over the chunk
        for (int tt = 0; tt < nt; ++tt) {
            const float* kr = k_s + tt * DP + rp * PS;
            const float* qr = q_s + tt * DP + rp * PS;
            const float* gr = g_s + tt * DP + rp * PS;
            float kreg[DPT];
            float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;         // four chains, so that no sum waits for the one before
#pragma unroll
            for (int ii = 0; ii < DPT; ii += 4) {
                const float4 k4 = *reinterpret_cast<const float4*>(kr + ii);
                const float4 g4 = *reinterpret_cast<const float4*>(gr + ii);
                kreg[ii] = k4.x; kreg[ii + 1] = k4.y; kreg[ii + 2] = k4.z; kreg[ii + 3] = k4.w;
                st[ii] *= g4.x; st[ii + 1] *= g4.y; st[ii + 2] *= g4.z; st[ii + 3] *= g4.w;
                a0 = fmaf(st[ii], k4.x, a0);
                a1 = fmaf(st[ii + 1], k4.y, a1);
                a2 = fmaf(st[ii + 2], k4.z, a2);
                a3 = fmaf(st[ii + 3], k4.w, a3);
            }
            const float acc = dr_group_sum((a0 + a1) + (a2 + a3), RS);
            const float u = beta_s[tt] * (v_s[tt * V + (live ? j : 0)] - acc);
            float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
#pragma unroll
            for (int ii = 0; ii < DPT; ii += 4) {
                const float4 q4 = *reinterpret_cast<const float4*>(qr + ii);
                st[ii] = fmaf(kreg[ii], u, st[ii]);
                st[ii + 1] = fmaf(kreg[ii + 1], u, st[ii + 1]);
                st[ii + 2] = fmaf(kreg[ii + 2], u, st[ii + 2]);
                st[ii + 3] = fmaf(kreg[ii + 3], u, st[ii + 3]);
                o0 = fmaf(st[ii], q4.x, o0);
                o1 = fmaf(st[ii + 1], q4.y, o1);
                o2 = fmaf(st[ii + 2], q4.z, o2);
                o3 = fmaf(st[ii + 3], q4.w, o3);
            }
            const float o = dr_group_sum((o0 + o1) + (o2 + o3), RS);
            if (live && rp == 0) o_s[tt * V + j] = o;
        }
        __syncthreads();
        // ---- norm over the head's read-out (a wave per row), then weight and output gate: a thread takes one
        // column of four rows at a time
        for (int tt = wave; tt < nt; tt += n_waves) {
            float ss = 0.f;
            for (int jj = lane; jj < V; jj += 64) ss = fmaf(o_s[tt * V + jj], o_s[tt * V + jj], ss);
            ss = wave_sum(ss);
            if (lane == 0) rstd_s[tt] = 1.0f / sqrtf(ss / (float)V + eps);
        }
        __syncthreads();
        for (int idx = tid; idx < ((nt + 3) >> 2) * V; idx += NT) {
            const int tg = idx / V, jj = idx - tg * V;
            float gt[4] = {0.f, 0.f, 0.f, 0.f};
            const float* g1 = g1_s + (tg * 4) * rgp;
#pragma unroll 2
            for (int r = 0; r < rgp; r += 4) {
                float w4[4];
#pragma unroll
                for (int x = 0; x < 4; ++x)
                    w4[x] = staged ? wg_s[(r + x) * V + jj]
                                   : (r + x < rg ? w_g2t[(size_t)(r + x) * H * V + h * V + jj] : 0.f);
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const float4 c4 = *reinterpret_cast<const float4*>(g1 + k * rgp + r);
                    gt[k] = fmaf(c4.x, w4[0], gt[k]);
                    gt[k] = fmaf(c4.y, w4[1], gt[k]);
                    gt[k] = fmaf(c4.z, w4[2], gt[k]);
                    gt[k] = fmaf(c4.w, w4[3], gt[k]);
                }
            }
            const float nw = norm_w[jj];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int tt = tg * 4 + k;
                if (tt >= nt) break;
                out[(size_t)(base + c0 + tt) * H * V + h * V + jj] =
                    from_f<T>(o_s[tt * V + jj] * rstd_s[tt] * nw * dr_sigmoid(gt[k]));
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int ii = 0; ii < DPT; ++ii) {
        const int i = rp * DPT + ii;
        if (live && i < D) Sh[(size_t)i * V + j] = st[ii];
    }
}

static size_t delta_rule_lds(int DPT, int RS, int V, int ra, int rg) {
    const int rap = (ra + 3) & ~3, rgp = (rg + 3) & ~3;
    return sizeof(float) * ((size_t)DR_TC * (3 * RS * (DPT + DR_PAD) + 2 * V + rap + rgp) + 2 * DR_TC);
}
// the low-rank factors' rows of one head beside that, if they fit
static size_t delta_rule_staged(int D, int V, int ra, int rg) {
    return sizeof(float) * ((size_t)((ra + 3) & ~3) * D + (size_t)((rg + 3) & ~3) * V);
}
#define DR_LDS_LIMIT (156 * 1024)

// The split of a column's rows over lanes: RS lanes (a power of two) of DPT rows each.
static bool delta_rule_plan(int D, int V, int* RS_out, int* DPT_out) {
    if (D < 1 || V < 1 || V > 512 || D > 512) return false;
    int RS = 8;
    while (RS > 1 && (V * RS > 512 || (D + RS - 1) / RS < 8)) RS >>= 1;
    const int need = (D + RS - 1) / RS;
    int DPT = 4;
    while (DPT < need) DPT <<= 1;
    if (DPT > 64) return false;
    *RS_out = RS;
    *DPT_out = DPT;
    return true;
}

extern "C" int ra_delta_rule_fits(int D, int V, int ra, int rg) {
    int RS, DPT;
    if (!delta_rule_plan(D, V, &RS, &DPT) || ra < 0 || rg < 0) return 0;
    return delta_rule_lds(DPT, RS, V, ra, rg) <= 160 * 1024 ? 1 : 0;
}

template <typename T>
static int delta_rule_launch(hipStream_t st, int DPT, dim3 grid, dim3 block, size_t lds, const void* qkv, long long ld_qkv,
                             const void* z, long long ld_z, int off_b, int off_a, int ra, int off_g, int rg,
                             const float* w_a2t, const float* w_g2t, const float* A_log, const float* dt_bias,
                             const float* norm_w, float eps, float* S, const int* cu_q, const int* slot_ids, void* out,
                             int H, int G, int D, int V, int RS, int staged) {
#define DR_GO(DPT_)                                                                                               \
    do {                                                                                                          \
        if (lds > 64 * 1024 &&                                                                                    \
            hipFuncSetAttribute((const void*)delta_rule_kernel<T, DPT_>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                (int)lds) != hipSuccess)                                                          \
            return RA_ERR_LAUNCH;                                                                                 \
        hipLaunchKernelGGL((delta_rule_kernel<T, DPT_>), grid, block, lds, st, (const T*)qkv, ld_qkv, (const T*)z, \
                           ld_z, off_b, off_a, ra, off_g, rg, w_a2t, w_g2t, A_log, dt_bias, norm_w, eps, S, cu_q,  \
                           slot_ids, (T*)out, H, G, D, V, RS, staged);                                            \
    } while (0)
    switch (DPT) {
        case 4: DR_GO(4); break;
        case 8: DR_GO(8); break;
        case 16: DR_GO(16); break;
        case 32: DR_GO(32); break;
        case 64: DR_GO(64); break;
        default: return RA_ERR_ARG;
    }
#undef DR_GO
    return ra_launch_status();
}

extern "C" int ra_delta_rule(const void* qkv, long long ld_qkv, const void* z, long long ld_z, int off_b, int off_a, int ra,
                             int off_g, int rg, const float* w_a2t, const float* w_g2t, const float* A_log,
                             const float* dt_bias, const float* norm_w, float eps, float* S, const int* cu_q,
                             const int* slot_ids, void* out, int n_seqs, int H, int G, int D, int V, int dtype,
                             void* stream) {
    if (n_seqs <= 0) return RA_OK;
    int RS, DPT;
    if (!delta_rule_plan(D, V, &RS, &DPT) || H < 1 || G < 1 || H % G || ra < 0 || rg < 0 || n_seqs > 65535) return RA_ERR_ARG;
    if (ld_qkv < (long long)2 * G * D + (long long)H * V || off_b < 0 || off_a < 0 || off_g < 0) return RA_ERR_ARG;
    if (ld_z < off_b + H || ld_z < off_a + ra || ld_z < off_g + rg) return RA_ERR_ARG;
    size_t lds = delta_rule_lds(DPT, RS, V, ra, rg);
    if (lds > 160 * 1024) return RA_ERR_ARG;
    const int staged = lds + delta_rule_staged(D, V, ra, rg) <= DR_LDS_LIMIT ? 1 : 0;
    if (staged) lds += delta_rule_staged(D, V, ra, rg);
    dim3 grid(H, n_seqs), block(((V * RS + 63) / 64) * 64);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == RA_DTYPE_F32)
        return delta_rule_launch<float>(st, DPT, grid, block, lds, qkv, ld_qkv, z, ld_z, off_b, off_a, ra, off_g, rg, w_a2t,
                                        w_g2t, A_log, dt_bias, norm_w, eps, S, cu_q, slot_ids, out, H, G, D, V, RS, staged);
    if (dtype == RA_DTYPE_BF16)
        return delta_rule_launch<bf16>(st, DPT, grid, block, lds, qkv, ld_qkv, z, ld_z, off_b, off_a, ra, off_g, rg, w_a2t,
                                       w_g2t, A_log, dt_bias, norm_w, eps, S, cu_q, slot_ids, out, H, G, D, V, RS, staged);
    return RA_ERR_ARG;
}
