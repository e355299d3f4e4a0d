// Differential attention over the paged cache: every query head has two score maps (two queries of size
// D against two keys of size D of its kv head), each a softmax attention of its own over the SAME values
// (size Dv), and the head's output is
//     o = a1 - lambda * a2;   o <- o / sqrt(mean(o^2) + eps) * out_scale      (norm over the head's Dv values)
// with one lambda for the layer. Rows of q are [Hq][2][D], rows of the key pool [2][D] per kv head (both
// maps of a token side by side, one read serves both), rows of the value pool [Dv].
//
// Masks: causal by position; window w (> 0): keys at positions > p - w; chunk c (> 0): keys at positions
// >= floor(p / c) * c, chunks counted from position 0 of the request. Both may be given.
//
// This file has the preparation kernel (rotation of both maps, q out, k and v into the pools) and the
// plain kernel: every product and sum a 32-bit FMA, any sizes, for the float32 path and for sizes the
// matrix-core kernel (attention_diff_mfma.hip) does not take. Tables as in attention_plain.hip.
#include "common.h"

// ------------------------------------------------------------------ preparation
// qkv row: [Hq*M*D | Hkv*M*D | Hkv*Dv] (M maps). The first R elements of every map of q and k are rotated
// by the token's position: interleaved (element 2i with 2i+1) or half-split (i with i + R/2); cos/sin are
// [positions][R/2] in 32-bit. q goes to q_out [T][Hq*M*D], k to the key pool row of the token's slot, v to
// the value pool row. A workgroup per token and 1,024 elements of its row.
template <typename T>
__global__ void maps_prepare_kernel(const T* __restrict__ qkv, int Hq, int Hkv, int M, int D, int Dv,
                                    const int* __restrict__ positions, const float* __restrict__ cos_t,
                                    const float* __restrict__ sin_t, int R, int interleaved,
                                    T* __restrict__ q_out, T* __restrict__ k_pool, T* __restrict__ v_pool,
                                    const int* __restrict__ slot_mapping, int P) {
    const int t = blockIdx.x;
    const int qw = Hq * M * D, kw = Hkv * M * D, vw = Hkv * Dv;
    const T* row = qkv + (size_t)t * (qw + kw + vw);
    const int pos = positions[t];
    const int half = R >> 1;
    const long long slot = slot_mapping ? slot_mapping[t] : 0;
    // (a workgroup takes 1,024 elements of the token's row, a thread four of them: their reads are asked for together)
    const int c_end = min(qw + kw + vw, ((int)blockIdx.y + 1) * 1024);
#pragma unroll 4
    for (int c = blockIdx.y * 1024 + threadIdx.x; c < c_end; c += 256) {
        if (c >= qw + kw) {                                   // a value
            if (v_pool == nullptr) continue;
            const int e = c - qw - kw, h = e / Dv;
            v_pool[ra_cache_offset(slot, h, Hkv, P, Dv) + (e - h * Dv)] = row[c];
            continue;
        }
        const int d = c % D;                                  // element within its map
        float x = to_f(row[c]);
        if (d < R) {
            int i, other;
            bool first;
            if (interleaved) { i = d >> 1; first = (d & 1) == 0; other = first ? c + 1 : c - 1; }
            else { first = d < half; i = first ? d : d - half; other = first ? c + half : c - half; }
            const float y = to_f(row[other]);
            const float cs = cos_t[(size_t)pos * half + i], sn = sin_t[(size_t)pos * half + i];
            x = first ? x * cs - y * sn : x * cs + y * sn;
        }
        if (c < qw) {
            q_out[(size_t)t * qw + c] = from_f<T>(x);
        } else if (k_pool != nullptr) {
            const int e = c - qw, h = e / (M * D);
            k_pool[ra_cache_offset(slot, h, Hkv, P, M * D) + (e - h * M * D)] = from_f<T>(x);
        }
    }
}

extern "C" int ra_maps_qkv_prepare(const void* qkv, int T_tokens, int Hq, int Hkv, int M, int D, int Dv,
                                   const int* positions, const float* cos_t, const float* sin_t, int R,
                                   int interleaved, void* q_out, void* k_pool, void* v_pool,
                                   const int* slot_mapping, int P, int dtype, void* stream) {
    if (T_tokens <= 0) return RA_OK;
    if (Hq <= 0 || Hkv <= 0 || M <= 0 || D <= 0 || Dv <= 0 || R < 0 || R > D || (R & 1) || P <= 0) return RA_ERR_ARG;
    if (R > 0 && (cos_t == nullptr || sin_t == nullptr)) return RA_ERR_ARG;
    if ((k_pool != nullptr || v_pool != nullptr) && slot_mapping == nullptr) return RA_ERR_ARG;
    const long long len = (long long)(Hq + Hkv) * M * D + (long long)Hkv * Dv;
    if (len > 65535LL * 1024) return RA_ERR_ARG;
    dim3 grid(T_tokens, (unsigned)((len + 1023) / 1024)), block(256);
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(maps_prepare_kernel<float>, grid, block, 0, (hipStream_t)stream, (const float*)qkv, Hq, Hkv,
                           M, D, Dv, positions, cos_t, sin_t, R, interleaved, (float*)q_out, (float*)k_pool,
                           (float*)v_pool, slot_mapping, P);
    else if (dtype == RA_DTYPE_BF16)
        hipLaunchKernelGGL(maps_prepare_kernel<bf16>, grid, block, 0, (hipStream_t)stream, (const bf16*)qkv, Hq, Hkv,
                           M, D, Dv, positions, cos_t, sin_t, R, interleaved, (bf16*)q_out, (bf16*)k_pool,
                           (bf16*)v_pool, slot_mapping, P);
    else
        return RA_ERR_ARG;
    return ra_launch_status();
}

// ------------------------------------------------------------------ the plain kernel
// A workgroup takes QR consecutive query rows of one head; rows of one request share a pass over the
// keys. Its waves take the blocks of 64 key positions in turn (block b, counted from position 0, is wave
// b % WAVES's), so a row's sums are formed in an order that depends on nothing but its own positions, and
// are merged through LDS in wave order. Within a block four lanes share a key (each a quarter of the
// elements of both maps), 16 keys at once; for the values the lanes run along the head's Dv elements.
#define DIFF_MAX_ACC 8      // Dv <= 64 * 8
#define DIFF_BLOCK 64

template <typename T, int QR, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void attn_diff_plain_kernel(
    const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ k_pool,
    const T* __restrict__ v_pool, const int* __restrict__ page_table,
    const int* __restrict__ cu_pages, const int* __restrict__ kv_start,
    const int* __restrict__ cu_q, const int* __restrict__ q_start,
    const int* __restrict__ tok_ids, int ids_are_requests, int n_seqs, int T_tokens, int Hq, int Hkv, int D, int Dv,
    int P, float scale, int window, int chunk, float lambda, float eps, float out_scale) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int D2 = 2 * D;
    float* q_s = smem;                                   // [QR][2D]
    float* p_s = q_s + QR * D2;                          // [WAVES][2][QR][64]
    int* row_s = (int*)(p_s + WAVES * 2 * QR * 64);      // [WAVES][64]
    float* ml_s = (float*)(row_s + WAVES * 64);          // [WAVES][2][QR][2]
    float* acc_s = ml_s + WAVES * 2 * QR * 2;            // [WAVES][2][QR][Dv]
    float* o_s = acc_s + (size_t)WAVES * 2 * QR * Dv;    // [QR][Dv]
    float* ss_s = o_s + QR * Dv;                         // [QR]

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, part = lane & 3, sub = lane >> 2;
    const int head = blockIdx.y, kvh = head / (Hq / Hkv);

    int t_of[QR], seg_of[QR], pos_of[QR];
    unsigned todo = 0;
#pragma unroll
    for (int r = 0; r < QR; ++r) {
        const int qi = blockIdx.x * QR + r;
        t_of[r] = seg_of[r] = pos_of[r] = 0;
        if (qi < T_tokens) {
            int t, lo;
            if (tok_ids != nullptr && ids_are_requests) {          // the list names requests that bring one token each
                lo = tok_ids[qi];
                t = cu_q[lo];
            } else {
                t = tok_ids ? tok_ids[qi] : qi;
                lo = 0;
                int hi = n_seqs - 1;
                while (lo < hi) {
                    const int mid = (lo + hi + 1) >> 1;
                    if (cu_q[mid] <= t) lo = mid; else hi = mid - 1;
                }
            }
            todo |= 1u << r;
            t_of[r] = t;
            seg_of[r] = lo;
            pos_of[r] = q_start[lo] + (t - cu_q[lo]);
        }
    }

    while (todo) {                                       // one pass per request among the rows; the same in every thread
        int s = 0;
#pragma unroll
        for (int r = QR - 1; r >= 0; --r)
            if ((todo >> r) & 1u) s = seg_of[r];
        bool active[QR];
        int first_of[QR];
        const int start = kv_start[s];
        int lo_pos = 0x7fffffff, hi_pos = -1;
#pragma unroll
        for (int r = 0; r < QR; ++r) {
            active[r] = ((todo >> r) & 1u) && seg_of[r] == s;
            if (active[r]) todo &= ~(1u << r);
            int f = start;
            if (window > 0) f = max(f, pos_of[r] - window + 1);
            if (chunk > 0) f = max(f, (pos_of[r] / chunk) * chunk);
            first_of[r] = f;
            if (active[r]) {
                lo_pos = min(lo_pos, f);
                hi_pos = max(hi_pos, pos_of[r]);
            }
        }
        const int* pt = page_table + cu_pages[s];
        const int n_listed = cu_pages[s + 1] - cu_pages[s];

#pragma unroll
        for (int r = 0; r < QR; ++r) {
            const T* qr = q + ((size_t)t_of[r] * Hq + head) * D2;
            for (int c = tid; c < D2; c += WAVES * 64) q_s[r * D2 + c] = active[r] ? to_f(qr[c]) : 0.f;
        }
        __syncthreads();

        float m[2][QR], l[2][QR], acc[2][QR][DIFF_MAX_ACC];
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int r = 0; r < QR; ++r) {
                m[a][r] = -INFINITY;
                l[a][r] = 0.f;
#pragma unroll
                for (int i = 0; i < DIFF_MAX_ACC; ++i) acc[a][r][i] = 0.f;
            }
        float* my_p = p_s + wave * 2 * QR * 64;
        int* my_row = row_s + wave * 64;

        const int b_first = lo_pos / DIFF_BLOCK;
        int b = b_first + ((wave - b_first) % WAVES + WAVES) % WAVES;      // first block >= b_first of this wave
        for (; b * DIFF_BLOCK <= hi_pos; b += WAVES) {
            const int base = b * DIFF_BLOCK;
            float sc[2][4][QR];
#pragma unroll
            for (int sp = 0; sp < 4; ++sp) {
                const int kk = 16 * sp + sub;
                const int p = base + kk;
                const int idx = p - start;
                const int pi = idx >= 0 ? idx / P : 0;
                const bool there = p >= lo_pos && p <= hi_pos && idx >= 0 && pi < n_listed;
                const int row = there ? (pt[pi] * Hkv + kvh) * P + (idx - pi * P) : -1;
                float dot[2][QR];
#pragma unroll
                for (int r = 0; r < QR; ++r) dot[0][r] = dot[1][r] = 0.f;
                if (there) {
                    const T* kr = k_pool + (size_t)row * D2;
#pragma unroll
                    for (int a = 0; a < 2; ++a)
                        for (int e = part; e < D; e += 4) {
                            const float kv = to_f(kr[a * D + e]);
#pragma unroll
                            for (int r = 0; r < QR; ++r) dot[a][r] = fmaf(q_s[r * D2 + a * D + e], kv, dot[a][r]);
                        }
                }
#pragma unroll
                for (int a = 0; a < 2; ++a)
#pragma unroll
                    for (int r = 0; r < QR; ++r) {
                        float d = dot[a][r];
                        d += __shfl_xor(d, 1, 64);
                        d += __shfl_xor(d, 2, 64);
                        const bool ok = there && active[r] && p <= pos_of[r] && p >= first_of[r];
                        sc[a][sp][r] = ok ? d * scale : -INFINITY;
                    }
                if (part == 0) my_row[kk] = row;
            }
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
                for (int r = 0; r < QR; ++r) {
                    const float mx = wave_max(fmaxf(fmaxf(sc[a][0][r], sc[a][1][r]), fmaxf(sc[a][2][r], sc[a][3][r])));
                    const float m_new = fmaxf(m[a][r], mx);
                    const float alpha = (m[a][r] == -INFINITY) ? 0.f : expf(m[a][r] - m_new);
                    float mine = 0.f;
#pragma unroll
                    for (int sp = 0; sp < 4; ++sp) {
                        const float pr = (sc[a][sp][r] == -INFINITY) ? 0.f : expf(sc[a][sp][r] - m_new);
                        if (part == 0) {
                            my_p[(a * QR + r) * 64 + 16 * sp + sub] = pr;
                            mine += pr;
                        }
                    }
                    l[a][r] = l[a][r] * alpha + wave_sum(mine);
                    m[a][r] = m_new;
#pragma unroll
                    for (int i = 0; i < DIFF_MAX_ACC; ++i) acc[a][r][i] *= alpha;
                }
            __builtin_amdgcn_wave_barrier();
            const int nk = min(DIFF_BLOCK, hi_pos - base + 1);
#pragma unroll 2
            for (int kk = 0; kk < nk; ++kk) {
                const int row = max(my_row[kk], 0);      // a key that is not there has probability 0
                const T* vr = v_pool + (size_t)row * Dv;
                float pv[2][QR];
#pragma unroll
                for (int a = 0; a < 2; ++a)
#pragma unroll
                    for (int r = 0; r < QR; ++r) pv[a][r] = my_p[(a * QR + r) * 64 + kk];
#pragma unroll
                for (int i = 0; i < DIFF_MAX_ACC; ++i) {
                    const int e = lane + 64 * i;
                    if (e < Dv) {
                        const float v = to_f(vr[e]);
#pragma unroll
                        for (int a = 0; a < 2; ++a)
#pragma unroll
                            for (int r = 0; r < QR; ++r) acc[a][r][i] = fmaf(pv[a][r], v, acc[a][r][i]);
                    }
                }
            }
            __builtin_amdgcn_wave_barrier();
        }

        // ---- merge of the waves, in wave order; then lambda, the head's norm and the factor
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int r = 0; r < QR; ++r) {
                if (lane == 0) {
                    ml_s[((wave * 2 + a) * QR + r) * 2] = m[a][r];
                    ml_s[((wave * 2 + a) * QR + r) * 2 + 1] = l[a][r];
                }
#pragma unroll
                for (int i = 0; i < DIFF_MAX_ACC; ++i) {
                    const int e = lane + 64 * i;
                    if (e < Dv) acc_s[(size_t)((wave * 2 + a) * QR + r) * Dv + e] = acc[a][r][i];
                }
            }
        __syncthreads();
        for (int idx = tid; idx < QR * Dv; idx += WAVES * 64) {
            const int r = idx / Dv, e = idx - r * Dv;
            float res[2];
#pragma unroll
            for (int a = 0; a < 2; ++a) {
                float mm = -INFINITY;
                for (int w = 0; w < WAVES; ++w) mm = fmaxf(mm, ml_s[((w * 2 + a) * QR + r) * 2]);
                float num = 0.f, den = 0.f;
                for (int w = 0; w < WAVES; ++w) {
                    const float mw = ml_s[((w * 2 + a) * QR + r) * 2];
                    const float ew = (mw == -INFINITY) ? 0.f : expf(mw - mm);
                    num = fmaf(acc_s[(size_t)((w * 2 + a) * QR + r) * Dv + e], ew, num);
                    den = fmaf(ml_s[((w * 2 + a) * QR + r) * 2 + 1], ew, den);
                }
                res[a] = den > 0.f ? num / den : 0.f;
            }
            o_s[idx] = res[0] - lambda * res[1];
        }
        __syncthreads();
        for (int r = wave; r < QR; r += WAVES) {         // a wave sums the squares of a row
            float ss = 0.f;
            for (int e = lane; e < Dv; e += 64) ss = fmaf(o_s[r * Dv + e], o_s[r * Dv + e], ss);
            ss = wave_sum(ss);
            if (lane == 0) ss_s[r] = ss;
        }
        __syncthreads();
        for (int idx = tid; idx < QR * Dv; idx += WAVES * 64) {
            const int r = idx / Dv, e = idx - r * Dv;
            bool act = false;
            int t_row = 0;
#pragma unroll
            for (int rr = 0; rr < QR; ++rr)
                if (rr == r) { act = active[rr]; t_row = t_of[rr]; }
            if (!act) continue;
            const float rstd = 1.0f / sqrtf(ss_s[r] / (float)Dv + eps);
            out[((size_t)t_row * Hq + head) * Dv + e] = from_f<T>(o_s[idx] * rstd * out_scale);
        }
        __syncthreads();                                 // before the next pass writes q_s and the merge buffers
    }
}

static size_t diff_plain_floats(int QR, int WAVES, int D, int Dv) {
    return (size_t)QR * 2 * D + (size_t)WAVES * 2 * QR * 64 + WAVES * 64 + (size_t)WAVES * 2 * QR * 2 +
           (size_t)WAVES * 2 * QR * Dv + (size_t)QR * Dv + QR;
}

template <typename T, int QR, int WAVES>
static void diff_plain_launch(hipStream_t st, const void* q, void* out, const void* k_pool, const void* v_pool,
                              const int* page_table, const int* cu_pages, const int* kv_start, const int* cu_q,
                              const int* q_start, const int* tok_ids, int ids_are_requests, int n_seqs, int T_tokens,
                              int Hq, int Hkv, int D, int Dv, int P, float scale, int window, int chunk, float lambda,
                              float eps, float out_scale) {
    dim3 grid((T_tokens + QR - 1) / QR, Hq), block(WAVES * 64);
    hipLaunchKernelGGL((attn_diff_plain_kernel<T, QR, WAVES>), grid, block, diff_plain_floats(QR, WAVES, D, Dv) * sizeof(float),
                       st, (const T*)q, (T*)out, (const T*)k_pool, (const T*)v_pool, page_table, cu_pages, kv_start,
                       cu_q, q_start, tok_ids, ids_are_requests, n_seqs, T_tokens, Hq, Hkv, D, Dv, P, scale, window, chunk,
                       lambda, eps, out_scale);
}

// Whether the plain kernel takes these sizes (its LDS holds a row's query maps and the waves' sums).
extern "C" int ra_attention_diff_plain_fits(int D, int Dv) {
    return D >= 1 && Dv >= 1 && Dv <= 64 * DIFF_MAX_ACC && diff_plain_floats(1, 4, D, Dv) * sizeof(float) <= 65536;
}

extern "C" int ra_attention_diff_plain(const void* q, void* out, const void* k_pool, const void* v_pool,
                                       const int* page_table, const int* cu_pages, const int* kv_start,
                                       const int* cu_q, const int* q_start, const int* tok_ids,
                                       int ids_are_requests, int n_seqs, int T_tokens, int Hq, int Hkv, int D, int Dv, int P, float scale, int window,
                                       int chunk, float lambda, float eps, float out_scale, int dtype, void* stream) {
    if (T_tokens <= 0 || n_seqs <= 0) return RA_OK;
    if (!ra_attention_diff_plain_fits(D, Dv) || Hkv <= 0 || Hq % Hkv != 0 || P <= 0 || Hq > 65535) return RA_ERR_ARG;
    if (dtype != RA_DTYPE_F32 && dtype != RA_DTYPE_BF16) return RA_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    // tok_ids: the rows of q to work on (null: all T_tokens rows), or, with ids_are_requests, the numbers of
    // requests that bring one token each (their rows are cu_q[request])
    const bool single = (tok_ids == nullptr && T_tokens == n_seqs) || (tok_ids != nullptr && ids_are_requests);
    const size_t limit = 65536 / sizeof(float);
#define DIFF_GO(T_, QR_, W_)                                                                                  \
    diff_plain_launch<T_, QR_, W_>(st, q, out, k_pool, v_pool, page_table, cu_pages, kv_start, cu_q, q_start,  \
                                   tok_ids, ids_are_requests, n_seqs, T_tokens, Hq, Hkv, D, Dv, P, scale, window, chunk,  \
                                   lambda, eps, out_scale)
#define DIFF_PICK(T_)                                                                                         \
    do {                                                                                                      \
        if (single && diff_plain_floats(1, 8, D, Dv) <= limit) DIFF_GO(T_, 1, 8);                             \
        else if (!single && diff_plain_floats(4, 4, D, Dv) <= limit) DIFF_GO(T_, 4, 4);                       \
        else if (!single && diff_plain_floats(2, 4, D, Dv) <= limit) DIFF_GO(T_, 2, 4);                       \
        else DIFF_GO(T_, 1, 4);                                                                               \
    } while (0)
    if (dtype == RA_DTYPE_F32) DIFF_PICK(float); else DIFF_PICK(bf16);
#undef DIFF_PICK
#undef DIFF_GO
    return ra_launch_status();
}
