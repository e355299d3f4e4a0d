// Differential attention on the matrix cores, bfloat16: the new tokens of a request, a portion of a prompt or
// a single token, over what the paged cache holds for it. The formulas, the masks (causal, window, chunk) and
// the tables are those of attention_diff.hip; sizes: a map of D = 16, 32, 48, 64, 96 or 128 elements,
// values of Dv = 32, 64, 96, 128, 192 or 256.
//
// BUILD-VARIANTS: DIFF_D16=1 DIFF_D16=2 DIFF_D16=3 DIFF_D16=4 DIFF_D16=6 DIFF_D16=8 DIFF_API=1
//
// One workgroup of four waves per (q tile of 64 rows, query head); wave w owns rows 16w .. 16w+15. Per pass
// a tile of BN keys sits in LDS: the key rows (both maps side by side) and the value rows, row-major with
// padded rows; the next tile's rows are on their way from the cache into registers while this one is used.
//  scores  S^T = K Q^T for each map by MFMA 16x16x32 bf16: A = 16 key rows from LDS, B = the wave's 16
//          query rows held in registers. Lane (n, g) gets query n, keys 4g..4g+3 of each 16-key tile.
//  softmax one running maximum and sum per map and row, the scale folded into the exponent.
//  P.V     O^T += V^T P^T for each map, P as the sum of two bfloat16 halves (two MFMAs), so that the weights
//          keep 16 bits of mantissa: the contraction runs over the keys in the order the lanes hold them
//          (k-slot (g, e) of a 32-key block is key 16*(e/4) + 4g + e%4), so P goes from the softmax registers
//          into the B operand; V^T comes from the row-major V tile through the transposing LDS read
//          (ds_read_b64_tr_b16) and serves both maps.
//  end     o = a1 / l1 - lambda a2 / l2 per element, the sum of squares over the head's Dv elements (in the
//          lane, then over the four lane groups), o * rsqrt(mean + eps) * out_scale.
#include "common.h"

typedef __bf16 dbf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 dbf16x2_t __attribute__((ext_vector_type(2)));
typedef short dshort4_t __attribute__((ext_vector_type(4)));
typedef short dshort8_t __attribute__((ext_vector_type(8)));
typedef float dfloat4_t __attribute__((ext_vector_type(4)));
typedef float dfloat2_t __attribute__((ext_vector_type(2)));
typedef uint32_t duint4_t __attribute__((ext_vector_type(4)));
typedef dshort4_t __attribute__((address_space(3))) * dlds_short4_ptr;

#ifdef DIFF_D16

__device__ __forceinline__ uint32_t dpack2(float a, float b) {
    const dfloat2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, dbf16x2_t));
}

// the earliest key that the query at position p reads
__device__ __forceinline__ int diff_first_key(int p, int start, int window, int chunk) {
    int f = start;
    if (window > 0) f = max(f, p - window + 1);
    if (chunk > 0) f = max(f, (p / chunk) * chunk);
    return f;
}

// PACK (tiles of one row: requests that bring one token): a workgroup takes a kv head and the rows of its first
// wave are the query heads of that kv head's group (up to 16), so the group's keys and values are read once.
// (One wave a workgroup, eight such workgroups a CU, was measured and is not faster: 77 against 65 us a layer at
// batch 8 over 2,048 keys.)
template <int D16, int DV16, int BN, bool PACK>
__global__ __launch_bounds__(256) void attn_diff_mfma_kernel(
    const bf16* __restrict__ q, bf16* __restrict__ out, const bf16* __restrict__ k_pool,
    const bf16* __restrict__ v_pool, const int* __restrict__ page_table,
    const int* __restrict__ cu_pages, const int* __restrict__ kv_start,
    const int* __restrict__ cu_q, const int* __restrict__ q_start,
    const int* __restrict__ tiles,       // [n_tiles][2]: request number, first row of the tile within it
    int n_tiles, int Hq, int Hkv, int P, float scale, int window, int chunk, float lambda, float eps,
    float out_scale, int n_splits, float* __restrict__ part) {
    constexpr int D = 16 * D16, DK = 2 * D, DV = 16 * DV16;
    constexpr int D32 = D / 32;
    constexpr bool TAIL16 = (D % 32) != 0;
    constexpr int KS = DK + 8;                          // K tile row stride (elements): rows shift by 4 banks
    constexpr int VS = DV + 16;                         // V tile row stride: rows shift by 8 banks (transposing reads)
    constexpr int LPRK = DK / 8, LPRV = DV / 8;         // 16-byte pieces in one row
    constexpr int NT = 256;                             // threads of the workgroup
    constexpr int NK = (BN * LPRK + NT - 1) / NT, NV = (BN * LPRV + NT - 1) / NT;     // pieces per thread per tile
    __shared__ __attribute__((aligned(16))) uint16_t k_s[BN * KS];
    __shared__ __attribute__((aligned(16))) uint16_t v_s[BN * VS];

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, n = lane & 15, g = lane >> 4;
    const int grp = Hq / Hkv;
    const int tile = PACK ? blockIdx.x / Hkv : blockIdx.x / Hq;
    const int kvh = PACK ? blockIdx.x % Hkv : (blockIdx.x % Hq) / grp;
    const int head = PACK ? kvh * grp + min(n, grp - 1) : blockIdx.x % Hq;     // (PACK: this lane's row is a head of its own)
    const int seg = tiles[2 * tile], q_off = tiles[2 * tile + 1];
    const int q_len = cu_q[seg + 1] - cu_q[seg];
    const int pos0 = q_start[seg];
    const int start = kv_start[seg];
    const int* pt = page_table + cu_pages[seg];

    // this lane's query row (for the B operands and for the mask): row n of the wave's 16
    const int q_local = PACK ? q_off : q_off + wave * 16 + n;
    const bool q_ok = PACK ? (wave == 0 && n < grp && q_local < q_len) : q_local < q_len;
    const int pos_q = pos0 + q_local;
    const int first_q = diff_first_key(pos_q, start, window, chunk);
    const dbf16x8_t z8 = {0, 0, 0, 0, 0, 0, 0, 0};
    dbf16x8_t bq[2][D32 > 0 ? D32 : 1], bq_tail[2];
    {
        const bf16* qp = q + ((size_t)(cu_q[seg] + (q_ok ? q_local : 0)) * Hq + head) * DK;
#pragma unroll
        for (int mp = 0; mp < 2; ++mp) {
#pragma unroll
            for (int j = 0; j < D32; ++j) {
                const dbf16x8_t v = *reinterpret_cast<const dbf16x8_t*>(qp + mp * D + 32 * j + 8 * g);
                bq[mp][j] = q_ok ? v : z8;
            }
            bq_tail[mp] = z8;
            if constexpr (TAIL16) {
                if (q_ok && g < 2) bq_tail[mp] = *reinterpret_cast<const dbf16x8_t*>(qp + mp * D + (D - 16) + 8 * g);
            }
        }
    }

    const int tile_first_pos = pos0 + q_off;
    const int tile_last_pos = pos0 + min(q_off + 64, q_len) - 1;
    const int low_key = diff_first_key(tile_first_pos, start, window, chunk);    // the earliest key any row reads
    const int u_first = (low_key / BN) * BN;
    // the wave's rows: positions, and the first keys of its first and last row (first keys rise with the position)
    const int wave_first_pos = tile_first_pos + wave * 16, wave_last_pos = PACK ? wave_first_pos : wave_first_pos + 15;
    const int wave_low = diff_first_key(wave_first_pos, start, window, chunk);
    const int wave_high = diff_first_key(wave_last_pos, start, window, chunk);

    const float scale2 = scale * 1.44269504088896340736f;
    float m_run[2] = {-INFINITY, -INFINITY}, l_run[2] = {0.f, 0.f};
    dfloat4_t acc[2][DV16];
#pragma unroll
    for (int mp = 0; mp < 2; ++mp)
#pragma unroll
        for (int dt = 0; dt < DV16; ++dt) acc[mp][dt] = dfloat4_t{0.f, 0.f, 0.f, 0.f};

    duint4_t kreg[NK], vreg[NV];
    const int p_shift = (P & (P - 1)) == 0 ? __builtin_ctz(P) : -1;
    // cache row of key position kp (clamped into what this tile may read, so every address is valid)
    auto row_of = [&](int kp) {
        const int idx = min(max(kp, low_key), tile_last_pos) - start;
        const int pi = p_shift >= 0 ? (idx >> p_shift) : (idx / P);
        return (pt[pi] * Hkv + kvh) * P + (idx - pi * P);
    };
    // The cache rows of a tile's pieces are looked up one pass before the pieces are asked for, so that a fetch
    // does not wait for the page table first (a read that waits for a read costs more than a pass's products).
    int rk[NK], rv[NV];
#define DIFF_ROWS(u_)                                                                     \
    {                                                                                     \
        _Pragma("unroll") for (int i = 0; i < NK; ++i) {                                  \
            const int pc = tid + NT * i;                                                  \
            rk[i] = pc < BN * LPRK ? row_of((u_) + pc / LPRK) : 0;                        \
        }                                                                                 \
        _Pragma("unroll") for (int i = 0; i < NV; ++i) {                                  \
            const int pc = tid + NT * i;                                                  \
            rv[i] = pc < BN * LPRV ? row_of((u_) + pc / LPRV) : 0;                        \
        }                                                                                 \
    }
#define DIFF_FETCH()                                                                      \
    {                                                                                     \
        _Pragma("unroll") for (int i = 0; i < NK; ++i) {                                  \
            const int pc = tid + NT * i;                                                  \
            if (pc < BN * LPRK)                                                           \
                kreg[i] = *reinterpret_cast<const duint4_t*>(k_pool + (size_t)rk[i] * DK + 8 * (pc % LPRK)); \
        }                                                                                 \
        _Pragma("unroll") for (int i = 0; i < NV; ++i) {                                  \
            const int pc = tid + NT * i;                                                  \
            if (pc < BN * LPRV)                                                           \
                vreg[i] = *reinterpret_cast<const duint4_t*>(v_pool + (size_t)rv[i] * DV + 8 * (pc % LPRV)); \
        }                                                                                 \
    }
#define DIFF_STAGE()                                                                      \
    {                                                                                     \
        _Pragma("unroll") for (int i = 0; i < NK; ++i) {                                  \
            const int pc = tid + NT * i;                                                  \
            if (pc < BN * LPRK) {                                                         \
                const int r_ = pc / LPRK, c_ = pc - r_ * LPRK;                            \
                *reinterpret_cast<duint4_t*>(k_s + r_ * KS + 8 * c_) = kreg[i];           \
            }                                                                             \
        }                                                                                 \
        _Pragma("unroll") for (int i = 0; i < NV; ++i) {                                  \
            const int pc = tid + NT * i;                                                  \
            if (pc < BN * LPRV) {                                                         \
                const int r_ = pc / LPRV, c_ = pc - r_ * LPRV;                            \
                *reinterpret_cast<duint4_t*>(v_s + r_ * VS + 8 * c_) = vreg[i];           \
            }                                                                             \
        }                                                                                 \
    }

    // With n_splits > 1 (tiles of one row: requests that bring one token) the workgroups blockIdx.y = 0, 1, ...
    // share the tile's key blocks evenly and leave their sums to the merge kernel.
    int u_lo = u_first, u_hi = tile_last_pos;            // first key block, and the last key, of this workgroup
    if (n_splits > 1) {
        const int blocks = (tile_last_pos - u_first) / BN + 1;
        const int per = (blocks + n_splits - 1) / n_splits;
        u_lo = u_first + (int)blockIdx.y * per * BN;
        u_hi = min(tile_last_pos, u_lo + per * BN - 1);
    }
    if (u_lo <= u_hi) {
        DIFF_ROWS(u_lo)
        DIFF_FETCH()
        DIFF_ROWS(u_lo + BN)                             // (beyond the last key the rows are clamped to valid ones)
    }
    for (int u = u_lo; u <= u_hi; u += BN) {
        __syncthreads();                                 // every wave is done with the tile before
        DIFF_STAGE()
        __syncthreads();
        if (u + BN <= u_hi) {                            // the next tile, on its way while this one is used
            DIFF_FETCH()
            DIFF_ROWS(u + 2 * BN)
        }

        // a tile that lies wholly above every row of the wave, or wholly before their first keys, has nothing for
        // it; nor has any tile for a wave whose rows all lie beyond the request's new tokens (a request that
        // brings one token: three waves only help to move the tiles)
        if (u <= wave_last_pos && u + BN - 1 >= wave_low && wave_first_pos <= tile_last_pos) {
            dfloat4_t cs[2][BN / 16];
#pragma unroll
            for (int st = 0; st < BN / 16; ++st) {
                const uint16_t* kr = &k_s[(st * 16 + n) * KS];
#pragma unroll
                for (int mp = 0; mp < 2; ++mp) {
                    cs[mp][st] = dfloat4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int j = 0; j < D32; ++j) {
                        const dbf16x8_t a = *reinterpret_cast<const dbf16x8_t*>(kr + mp * D + 32 * j + 8 * g);
                        cs[mp][st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bq[mp][j], cs[mp][st], 0, 0, 0);
                    }
                    if constexpr (TAIL16) {
                        dbf16x8_t a = z8;
                        if (g < 2) a = *reinterpret_cast<const dbf16x8_t*>(kr + mp * D + (D - 16) + 8 * g);
                        cs[mp][st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bq_tail[mp], cs[mp][st], 0, 0, 0);
                    }
                }
            }
            MFMA_SETTLE();
            // a tile that every row of the wave reads whole needs no mask
            const bool need_mask = (u + BN - 1 > wave_first_pos) || (u < wave_high);
            duint4_t pw[2][BN / 32], pl[2][BN / 32];             // the weights' upper and lower halves, in the order the B operand wants
#pragma unroll
            for (int mp = 0; mp < 2; ++mp) {
                float s[BN / 16][4];
                float mx = -INFINITY;
                // (two branches, as in the prefill kernel of the ordinary attention: the one-branch form
                // "unmasked or visible" came out of the compiler with the first key of the first map masked)
                if (need_mask) {
#pragma unroll
                    for (int st = 0; st < BN / 16; ++st)
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const int kpos = u + st * 16 + 4 * g + i;
                            const bool ok = kpos >= first_q && kpos <= pos_q;
                            s[st][i] = ok ? cs[mp][st][i] : -INFINITY;
                            mx = fmaxf(mx, s[st][i]);
                        }
                } else {
#pragma unroll
                    for (int st = 0; st < BN / 16; ++st)
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            s[st][i] = cs[mp][st][i];
                            mx = fmaxf(mx, s[st][i]);
                        }
                }
                mx = rows_max(mx);
                const float m_new = fmaxf(m_run[mp], mx);
                const float m_use = (m_new == -INFINITY) ? 0.f : m_new;      // a row that sees no key yet keeps m = -inf
                const float off = -m_use * scale2;
                float lsum = 0.f;
#pragma unroll
                for (int st = 0; st < BN / 16; ++st)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        s[st][i] = __builtin_amdgcn_exp2f(fmaf(s[st][i], scale2, off));      // 2^(-inf) = 0 for masked keys
                        lsum += s[st][i];
                    }
                lsum = rows_sum(lsum);
                const float alpha = (m_run[mp] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((m_run[mp] - m_use) * scale2);
                l_run[mp] = l_run[mp] * alpha + lsum;
                if (__any(m_new != m_run[mp])) {
#pragma unroll
                    for (int dt = 0; dt < DV16; ++dt) {
                        acc[mp][dt][0] *= alpha;
                        acc[mp][dt][1] *= alpha;
                        acc[mp][dt][2] *= alpha;
                        acc[mp][dt][3] *= alpha;
                    }
                }
                m_run[mp] = m_new;
                // the weights go into the product as two bfloat16 numbers each, p = hi + lo (16 bits of mantissa
                // between them): the product's operands are 16-bit, the weights are not rounded to that
#pragma unroll
                for (int b = 0; b < BN / 32; ++b) {
                    const duint4_t hi = duint4_t{dpack2(s[2 * b][0], s[2 * b][1]), dpack2(s[2 * b][2], s[2 * b][3]),
                                                 dpack2(s[2 * b + 1][0], s[2 * b + 1][1]), dpack2(s[2 * b + 1][2], s[2 * b + 1][3])};
                    pw[mp][b] = hi;
                    float r[8];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        r[2 * e] = s[2 * b + e / 2][2 * (e & 1)] - __uint_as_float(hi[e] << 16);
                        r[2 * e + 1] = s[2 * b + e / 2][2 * (e & 1) + 1] - __uint_as_float(hi[e] & 0xffff0000u);
                    }
                    pl[mp][b] = duint4_t{dpack2(r[0], r[1]), dpack2(r[2], r[3]), dpack2(r[4], r[5]), dpack2(r[6], r[7])};
                }
            }
            // ---- O^T += V^T P^T, 32 keys per MFMA; V^T through the transposing LDS read, once for both maps
#pragma unroll
            for (int b = 0; b < BN / 32; ++b) {
                // this lane's address as lane l' = n of its group: key 32b + 4g + n/4, columns 4(n%4)..+3
                const uint16_t* vr = &v_s[(32 * b + 4 * g + (n >> 2)) * VS + 4 * (n & 3)];
#pragma unroll
                for (int dt = 0; dt < DV16; ++dt) {
                    const dshort4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((dlds_short4_ptr)(vr + dt * 16));
                    const dshort4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((dlds_short4_ptr)(vr + 16 * VS + dt * 16));
                    const dshort8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
                    for (int mp = 0; mp < 2; ++mp) {
                        acc[mp][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            __builtin_bit_cast(dbf16x8_t, both), __builtin_bit_cast(dbf16x8_t, pl[mp][b]), acc[mp][dt], 0, 0, 0);
                        acc[mp][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            __builtin_bit_cast(dbf16x8_t, both), __builtin_bit_cast(dbf16x8_t, pw[mp][b]), acc[mp][dt], 0, 0, 0);
                    }
                }
            }
        }
    }
#undef DIFF_FETCH
#undef DIFF_ROWS
#undef DIFF_STAGE
    MFMA_SETTLE();
    // ---- acc[mp][dt][i] = O^T[d = 16dt + 4g + i][query n]
    if (n_splits > 1) {
        // the tile's one row is lane n = 0 of wave 0: per map the running maximum (a raw score), the sum and
        // the unnormed row
        if (PACK ? q_ok : (wave == 0 && n == 0)) {
            float* pp = part + (((size_t)tile * Hq + head) * n_splits + blockIdx.y) * 2 * (DV + 2);
#pragma unroll
            for (int mp = 0; mp < 2; ++mp) {
                float* pm = pp + mp * (DV + 2);
                if (g == 0) {
                    pm[0] = m_run[mp];
                    pm[1] = l_run[mp];
                }
#pragma unroll
                for (int dt = 0; dt < DV16; ++dt)
                    *reinterpret_cast<dfloat4_t*>(pm + 2 + dt * 16 + 4 * g) = acc[mp][dt];
            }
        }
        return;
    }
    const float inv1 = l_run[0] > 0.f ? 1.0f / l_run[0] : 0.f;
    const float inv2 = l_run[1] > 0.f ? lambda / l_run[1] : 0.f;
    float ss = 0.f;
#pragma unroll
    for (int dt = 0; dt < DV16; ++dt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float o = acc[0][dt][i] * inv1 - acc[1][dt][i] * inv2;
            acc[0][dt][i] = o;
            ss = fmaf(o, o, ss);
        }
    ss = rows_sum(ss);                                   // the four lane groups hold the four quarters of the row
    const float f = out_scale / sqrtf(ss / (float)DV + eps);
    if (!q_ok) return;
    bf16* op = out + ((size_t)(cu_q[seg] + q_local) * Hq + head) * DV;
#pragma unroll
    for (int dt = 0; dt < DV16; ++dt) {
        uint2 w;
        w.x = dpack2(acc[0][dt][0] * f, acc[0][dt][1] * f);
        w.y = dpack2(acc[0][dt][2] * f, acc[0][dt][3] * f);
        *reinterpret_cast<uint2*>(op + dt * 16 + 4 * g) = w;
    }
}

#define DIFF_CAT2(a, b) a##b
#define DIFF_CAT(a, b) DIFF_CAT2(a, b)
#define DIFF_PART_ARGS int DV16, dim3 grid, hipStream_t st, const bf16* q, bf16* out, const bf16* kp, const bf16* vp,   \
    const int* pt, const int* cup, const int* kvs, const int* cuq, const int* qs, const int* tiles, int n_tiles, int Hq,  \
    int Hkv, int P, float scale, int window, int chunk, float lambda, float eps, float out_scale, int n_splits, float* part, \
    int pack
extern "C" int DIFF_CAT(ra_diff_part_, DIFF_D16)(DIFF_PART_ARGS) {
    // 64 keys a pass while a tile of them fits 40 KB of LDS, else 32
#define DIFF_CASE(V_)                                                                                           \
    case V_: {                                                                                                  \
        constexpr int BN_ = (64 * (2 * 16 * DIFF_D16 + 8 + 16 * V_ + 16) * 2 <= 40960) ? 64 : 32;               \
        if (pack)                                                                                               \
            hipLaunchKernelGGL((attn_diff_mfma_kernel<DIFF_D16, V_, BN_, true>), grid, dim3(256), 0, st, q, out, kp, vp, pt, \
                               cup, kvs, cuq, qs, tiles, n_tiles, Hq, Hkv, P, scale, window, chunk, lambda, eps,  \
                               out_scale, n_splits, part);                                                      \
        else                                                                                                    \
            hipLaunchKernelGGL((attn_diff_mfma_kernel<DIFF_D16, V_, BN_, false>), grid, dim3(256), 0, st, q, out, kp, vp, pt, \
                               cup, kvs, cuq, qs, tiles, n_tiles, Hq, Hkv, P, scale, window, chunk, lambda, eps,  \
                               out_scale, n_splits, part);                                                      \
        return RA_OK;                                                                                           \
    }
    switch (DV16) {
        DIFF_CASE(2) DIFF_CASE(4) DIFF_CASE(6) DIFF_CASE(8) DIFF_CASE(12) DIFF_CASE(16)
        default: return RA_ERR_ARG;
    }
#undef DIFF_CASE
}
#endif  // DIFF_D16

#ifdef DIFF_API
#define DIFF_PART_ARGS int DV16, dim3 grid, hipStream_t st, const bf16* q, bf16* out, const bf16* kp, const bf16* vp,   \
    const int* pt, const int* cup, const int* kvs, const int* cuq, const int* qs, const int* tiles, int n_tiles, int Hq,  \
    int Hkv, int P, float scale, int window, int chunk, float lambda, float eps, float out_scale, int n_splits, float* part, \
    int pack
extern "C" int ra_diff_part_1(DIFF_PART_ARGS);
extern "C" int ra_diff_part_2(DIFF_PART_ARGS);
extern "C" int ra_diff_part_3(DIFF_PART_ARGS);
extern "C" int ra_diff_part_4(DIFF_PART_ARGS);
extern "C" int ra_diff_part_6(DIFF_PART_ARGS);
extern "C" int ra_diff_part_8(DIFF_PART_ARGS);

// Whether the matrix-core kernel takes a map of D and values of Dv.
extern "C" int ra_attention_diff_mfma_fits(int D, int Dv) {
    const int d16 = D / 16, v16 = Dv / 16;
    if (D % 16 || Dv % 16) return 0;
    const bool d_ok = d16 == 1 || d16 == 2 || d16 == 3 || d16 == 4 || d16 == 6 || d16 == 8;
    const bool v_ok = v16 == 2 || v16 == 4 || v16 == 6 || v16 == 8 || v16 == 12 || v16 == 16;
    return d_ok && v_ok;
}

// The sums of a one-row tile's splits into its output row: per map the splits' maxima, sums and unnormed rows
// are merged in split order; then lambda, the head's norm and the factor. One wave per (tile, head).
__global__ __launch_bounds__(64) void attn_diff_merge_kernel(const float* __restrict__ part, bf16* __restrict__ out,
                                                             const int* __restrict__ tiles, const int* __restrict__ cu_q,
                                                             int Hq, int DV, int n_splits, float scale, float lambda,
                                                             float eps, float out_scale) {
    const int tile = blockIdx.x / Hq, head = blockIdx.x % Hq, lane = threadIdx.x;
    const float scale2 = scale * 1.44269504088896340736f;
    const float* pp = part + (size_t)blockIdx.x * n_splits * 2 * (DV + 2);
    float o[4] = {0.f, 0.f, 0.f, 0.f};                   // elements lane, lane + 64, ... (DV <= 256)
    const int token_row = cu_q[tiles[2 * tile]];         // (asked for now: a read that waits for a read is the time here)
    // lane sp reads split sp's maximum and sum of both maps (n_splits <= 64), all at once
    float my_m[2], my_l[2];
#pragma unroll
    for (int mp = 0; mp < 2; ++mp) {
        const float* mine = pp + ((size_t)min(lane, n_splits - 1) * 2 + mp) * (DV + 2);
        my_m[mp] = lane < n_splits ? mine[0] : -INFINITY;
        my_l[mp] = lane < n_splits ? mine[1] : 0.f;
    }
    float my_w[2], l[2] = {0.f, 0.f}, a[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
#pragma unroll
    for (int mp = 0; mp < 2; ++mp) {
        const float m = wave_max(my_m[mp]);
        my_w[mp] = (my_m[mp] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((my_m[mp] - m) * scale2);
    }
    for (int s0 = 0; s0 < n_splits; s0 += 8) {           // eight splits' rows of both maps asked for at once
        float raw[8][2][4];
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
            for (int mp = 0; mp < 2; ++mp) {
                const float* pm = pp + ((size_t)min(s0 + j, n_splits - 1) * 2 + mp) * (DV + 2);
#pragma unroll
                for (int i = 0; i < 4; ++i) raw[j][mp][i] = lane + 64 * i < DV ? pm[2 + lane + 64 * i] : 0.f;
            }
#pragma unroll
        for (int j = 0; j < 8; ++j) {                    // in split order
            if (s0 + j >= n_splits) break;
#pragma unroll
            for (int mp = 0; mp < 2; ++mp) {
                const float wgt = __shfl(my_w[mp], s0 + j, 64);
                l[mp] = fmaf(__shfl(my_l[mp], s0 + j, 64), wgt, l[mp]);
#pragma unroll
                for (int i = 0; i < 4; ++i) a[mp][i] = fmaf(raw[j][mp][i], wgt, a[mp][i]);
            }
        }
    }
#pragma unroll
    for (int mp = 0; mp < 2; ++mp) {
        const float f = l[mp] > 0.f ? (mp == 0 ? 1.0f : -lambda) / l[mp] : 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = fmaf(a[mp][i], f, o[i]);
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (lane + 64 * i < DV) ss = fmaf(o[i], o[i], ss);
    ss = wave_sum(ss);
    const float f = out_scale / sqrtf(ss / (float)DV + eps);
    bf16* op = out + ((size_t)token_row * Hq + head) * DV;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (lane + 64 * i < DV) op[lane + 64 * i] = from_f<bf16>(o[i] * f);
}

// floats of the buffer that n_splits > 1 needs for n_tiles one-row tiles
extern "C" long long ra_attention_diff_mfma_part_floats(int n_tiles, int Hq, int Dv, int n_splits) {
    return (long long)n_tiles * Hq * n_splits * 2 * (Dv + 2);
}

// tiles: int32 [n_tiles][2] = (request number, first row of the tile within the request's new tokens), tiles
// of 64 rows over the requests to work on (a request that brings one token is one tile with one row).
// n_splits > 1: every tile has ONE row (requests that bring one token), its keys are shared among n_splits
// workgroups whose sums go through part (ra_attention_diff_mfma_part_floats floats) and the merge kernel.
// pack (one-row tiles, at most 16 query heads a kv head): a workgroup per kv head works on all heads of its group.
extern "C" int ra_attention_diff_mfma_bf16(const void* q, void* out, const void* k_pool, const void* v_pool,
                                           const int* page_table, const int* cu_pages, const int* kv_start,
                                           const int* cu_q, const int* q_start, const int* tiles, int n_tiles,
                                           int Hq, int Hkv, int D, int Dv, int P, float scale, int window, int chunk,
                                           float lambda, float eps, float out_scale, int n_splits, float* part,
                                           int pack, void* stream) {
    if (n_tiles <= 0) return RA_OK;
    if (!ra_attention_diff_mfma_fits(D, Dv) || Hkv <= 0 || Hq % Hkv != 0 || P <= 0 || n_splits < 1 || n_splits > 65535 ||
        (n_splits > 1 && part == nullptr) || (long long)n_tiles * Hq > 0x7fffffffLL || (pack && Hq / Hkv > 16))
        return RA_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    dim3 grid(n_tiles * (pack ? Hkv : Hq), n_splits);
    int rc;
#define DIFF_GO(k)                                                                                            \
    rc = ra_diff_part_##k(Dv / 16, grid, st, (const bf16*)q, (bf16*)out, (const bf16*)k_pool, (const bf16*)v_pool, \
                          page_table, cu_pages, kv_start, cu_q, q_start, tiles, n_tiles, Hq, Hkv, P, scale, window, \
                          chunk, lambda, eps, out_scale, n_splits, part, pack)
    switch (D / 16) {
        case 1: DIFF_GO(1); break;
        case 2: DIFF_GO(2); break;
        case 3: DIFF_GO(3); break;
        case 4: DIFF_GO(4); break;
        case 6: DIFF_GO(6); break;
        case 8: DIFF_GO(8); break;
        default: return RA_ERR_ARG;
    }
#undef DIFF_GO
    if (rc != RA_OK) return rc;
    if (n_splits > 1)
        hipLaunchKernelGGL(attn_diff_merge_kernel, dim3(n_tiles * Hq), dim3(64), 0, st, part, (bf16*)out, tiles, cu_q, Hq,
                           Dv, n_splits, scale, lambda, eps, out_scale);
    return ra_launch_status();
}
#endif  // DIFF_API
