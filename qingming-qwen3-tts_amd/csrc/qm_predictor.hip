// qm_predictor.hip — the code predictor's whole per-frame attention loop in one launch (gfx950).
//
// One block owns one (unit, kv head), unit = (frame, layer): it stages the unit's 16 rows of
// Q (two heads), K and V in LDS (16 KiB), applies QK-RMSNorm + RoPE in place, then evaluates
// the 16 causal steps (row r attends keys 0..r) and writes the 16 context rows.  K/V never go
// back to HBM unless the caller asks for the cache.  Launch overhead is paid once for all
// frames, layers and steps instead of ~150 launches per frame.
//
// This operator keeps the reference's complete rounding chain, bf16(P) included, and its fp32
// summation topology (R17:12386-12418 dot products, 12449-12509 softmax, 12515-12574 P.V), so the
// result differs from the CPU restatement only where the device expf rounds differently.
//
// Algorithmic HBM bytes per (unit, kv head): 8 KiB q + 4 KiB k + 4 KiB v in, 8 KiB context out
// (+ 8 KiB if the K/V cache is written back) — the loop is bound by HBM bandwidth / latency.

#include "qm_device.h"
#include "qm_host.h"
#include "qm_predictor_params.h"
#include "qm_predictor_chain.h"

#include <type_traits>

namespace qm {

template <int R>
__device__ __forceinline__ void pv_rows(const float (*p)[kPredRows], const float* vcol, uint16_t* out,
                                        int64_t row_stride, int rows) {
    if constexpr (R < kPredRows) {
        if (R < rows) {
            const float* pr = p[R];
            // leaf j = fmaf(P[j], V[j][d], +0), keys 0..R (R17:12523-12549)
            const float o = TreeSum<R + 1, 0, 1>::eval([&](int j) { return fmaf(pr[j], vcol[j], 0.0f); });
            out[R * row_stride] = __builtin_bit_cast(uint16_t, static_cast<__bf16>(o));   // RNE, one instruction
            pv_rows<R + 1>(p, vcol, out, row_stride, rows);
        }
    }
}

// MODE 0: the loop (all rows of a unit from the projections' outputs).  MODE 1 (STAGED): attention only, over
// rotated queries and the caches.  MODE 2 (APPEND): one M = 1 step of a layer in one launch, what the
// reference runs as qk_norm_rope_cache_m1 + attention_m1 (R17:13700-13760): q [16][128], k, v [8][128] come from
// the projections, the caches [8][16][128] hold the rows before key_length - 1; the new K row (normed,
// rotated) and V row are written to the caches at key_length - 1 and the query attends key_length keys.
template <int MODE>
__global__ __launch_bounds__(kPredThreads) void predictor_loop_kernel(PredictorParams prm) {
    request_arguments(prm);
    constexpr bool STAGED = MODE == 1;
    constexpr bool APPEND = MODE == 2;
    __shared__ __attribute__((aligned(16))) uint16_t sh_q[2][kPredRows][kDim];   // [g][row][d]
    __shared__ __attribute__((aligned(16))) uint16_t sh_k[kPredRows][kDim];
    __shared__ __attribute__((aligned(16))) uint16_t sh_v[kPredRows][kDim];
    __shared__ __attribute__((aligned(16))) uint16_t sh_cos[kPredRows][kDim];
    __shared__ __attribute__((aligned(16))) uint16_t sh_sin[kPredRows][kDim];
    __shared__ __attribute__((aligned(16))) uint16_t sh_gamma[2][kDim];          // q, k
    __shared__ __attribute__((aligned(16))) float sh_s[2][kPredRows][kPredRows];   // scores, then P
    __shared__ __attribute__((aligned(16))) float sh_kf[kPredRows][kDim];                                       // normed, rotated K as fp32
    __shared__ float sh_grp[3 * kPredRows][4];                                     // group sums of squares
    __shared__ float sh_r[3 * kPredRows];                                          // inverse RMS per vector

    const int kvh = blockIdx.x;
    const int64_t unit = blockIdx.y;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int rows = prm.rows;
    const int layer = static_cast<int>((prm.unit_base + unit) % prm.n_layers);

    // keys row r attends: a prefix of the cache
    auto limit_of = [&](int r) {
        return STAGED ? (prm.causal ? min(r + 1, prm.key_length) : prm.key_length) : (APPEND ? prm.key_length : r + 1);
    };
    const int new_row = APPEND ? prm.key_length - 1 : 0;                 // APPEND: the cache row this step fills
    auto key_row_of = [&](int vrow) { return APPEND ? new_row : vrow; };   // where row vrow's K vector lives in sh_k
    if (STAGED) {
        // ---- q [16][rows][128] of this head pair, K and V rows 0..key_length-1 of the cache ------------
        for (int c = tid; c < rows * 32; c += kPredThreads) {
            const int chunk = c & 15, g = (c >> 4) & 1, row = c >> 5;
            *reinterpret_cast<uint4*>(&sh_q[g][row][chunk * 8]) = *reinterpret_cast<const uint4*>(
                prm.q + ((static_cast<int64_t>(kvh * 2 + g) * rows + row) * kDim) + chunk * 8);
        }
        for (int c = tid; c < kPredRows * 32; c += kPredThreads) {
            const int chunk = c & 15, is_v = (c >> 4) & 1, row = c >> 5;
            uint4 val = make_uint4(0, 0, 0, 0);
            if (row < prm.key_length)
                val = *reinterpret_cast<const uint4*>((is_v ? prm.v : prm.k) + (static_cast<int64_t>(kvh) * kPredRows + row) * kDim + chunk * 8);
            *reinterpret_cast<uint4*>(is_v ? &sh_v[row][chunk * 8] : &sh_k[row][chunk * 8]) = val;
        }
        __syncthreads();
        for (int c = tid; c < kPredRows * 32; c += kPredThreads) {
            const int row = c >> 5, d0 = (c & 31) * 4;
            const uint2 kk = *reinterpret_cast<const uint2*>(&sh_k[row][d0]);
            *reinterpret_cast<float4*>(&sh_kf[row][d0]) = make_float4(lo_bf16(kk.x), hi_bf16(kk.x), lo_bf16(kk.y), hi_bf16(kk.y));
        }
        __syncthreads();
    }
    if (APPEND) {
        // ---- the step's q (2 heads), k, v, its RoPE row and the gammas; the cache rows before it ----------
        for (int c = tid; c < 128; c += kPredThreads) {
            const int chunk = c & 15, which = c >> 4;     // 0,1: q head g; 2: k; 3: v; 4,5: cos, sin; 6,7: gammas
            const uint16_t* src = which < 2 ? prm.q + (kvh * 2 + which) * kDim
                                : which == 2 ? prm.k + kvh * kDim
                                : which == 3 ? prm.v + kvh * kDim
                                : which == 4 ? prm.cos_rows : which == 5 ? prm.sin_rows
                                : which == 6 ? prm.q_norm_w : prm.k_norm_w;
            uint16_t* dst = which < 2 ? sh_q[which][0] : which == 2 ? sh_k[new_row] : which == 3 ? sh_v[new_row]
                          : which == 4 ? sh_cos[0] : which == 5 ? sh_sin[0] : sh_gamma[which - 6];
            *reinterpret_cast<uint4*>(dst + chunk * 8) = *reinterpret_cast<const uint4*>(src + chunk * 8);
        }
        for (int c = tid; c < kPredRows * 32; c += kPredThreads) {
            const int chunk = c & 15, is_v = (c >> 4) & 1, row = c >> 5;
            if (row == new_row) continue;
            uint4 val = make_uint4(0, 0, 0, 0);
            if (row < new_row)
                val = *reinterpret_cast<const uint4*>((is_v ? prm.v_cache_out : prm.k_cache_out)
                                                      + (static_cast<int64_t>(kvh) * kPredRows + row) * kDim + chunk * 8);
            *reinterpret_cast<uint4*>(is_v ? &sh_v[row][chunk * 8] : &sh_k[row][chunk * 8]) = val;
        }
        __syncthreads();
        // (the new row is widened after its rotation, below)
        for (int c = tid; c < kPredRows * 32; c += kPredThreads) {
            const int row = c >> 5, d0 = (c & 31) * 4;
            if (row == new_row) continue;
            const uint2 kk = *reinterpret_cast<const uint2*>(&sh_k[row][d0]);
            *reinterpret_cast<float4*>(&sh_kf[row][d0]) = make_float4(lo_bf16(kk.x), hi_bf16(kk.x), lo_bf16(kk.y), hi_bf16(kk.y));
        }
    }
    if (MODE == 0) {
    // ---- stage q (2 heads), k, v of this kv head, the RoPE rows and the two gammas: 16-byte chunks ---
    for (int c = tid; c < rows * 64; c += kPredThreads) {
        const int chunk = c & 15;
        const int which = (c >> 4) & 3;     // 0,1: q head g; 2: k; 3: v
        const int row = c >> 6;
        const int64_t r64 = unit * rows + row;
        if (which < 2) {
            const uint4 val = *reinterpret_cast<const uint4*>(
                prm.q + ((r64 * 16 + kvh * 2 + which) * kDim) + chunk * 8);
            *reinterpret_cast<uint4*>(&sh_q[which][row][chunk * 8]) = val;
        } else {
            const uint16_t* src = which == 2 ? prm.k : prm.v;
            const uint4 val = *reinterpret_cast<const uint4*>(src + ((r64 * 8 + kvh) * kDim) + chunk * 8);
            *reinterpret_cast<uint4*>(which == 2 ? &sh_k[row][chunk * 8] : &sh_v[row][chunk * 8]) = val;
        }
    }
    for (int c = tid; c < rows * 32 + 32; c += kPredThreads) {
        const int chunk = c & 15;
        if (c < rows * 32) {
            const int row = c >> 5;
            const bool is_sin = (c >> 4) & 1;
            const uint4 val = *reinterpret_cast<const uint4*>((is_sin ? prm.sin_rows : prm.cos_rows) + row * kDim + chunk * 8);
            *reinterpret_cast<uint4*>(is_sin ? &sh_sin[row][chunk * 8] : &sh_cos[row][chunk * 8]) = val;
        } else {
            const int which = (c - rows * 32) >> 4;
            const uint4 val = *reinterpret_cast<const uint4*>((which ? prm.k_norm_w : prm.q_norm_w) + layer * kDim + chunk * 8);
            *reinterpret_cast<uint4*>(&sh_gamma[which][chunk * 8]) = val;
        }
    }
    __syncthreads();
    }   // MODE == 0
    if (!STAGED) {

    // ---- QK-RMSNorm + RoPE in place over the 3*rows head vectors (2 q heads + k per row) --------------
    // (1) One thread per (vector, 32-dim group): the group's sum of squares in the order of the
    //     reference's 32-lane shuffle tree (R17:8233-8245): x[i] + x[i+16], then +8, +4, +2, +1.
    const int n_vec = 3 * rows;
    for (int it = tid; it < n_vec * 4; it += kPredThreads) {
        const int vec = it >> 2, grp = it & 3;
        const int vrow = vec / 3, which = vec % 3;
        const uint16_t* x = (which < 2 ? sh_q[which][vrow] : sh_k[key_row_of(vrow)]) + 32 * grp;
        float sq[32];
#pragma unroll
        for (int i = 0; i < 32; i += 8) {
            const uint4 raw = *reinterpret_cast<const uint4*>(x + i);
            const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float a = lo_bf16(w[j]), b = hi_bf16(w[j]);
                sq[i + 2 * j] = a * a;
                sq[i + 2 * j + 1] = b * b;
            }
        }
#pragma unroll
        for (int stride = 16; stride > 0; stride >>= 1)
#pragma unroll
            for (int i = 0; i < stride; ++i) sq[i] = sq[i] + sq[i + stride];
        sh_grp[vec][grp] = sq[0];
    }
    __syncthreads();
    // (2) One thread per vector: (w0 + w2) + (w1 + w3), the reference's tree over the wave sums
    //     (R17:8262-8271), then 1 / sqrt(mean + eps).
    if (tid < n_vec) {
        const float total = (sh_grp[tid][0] + sh_grp[tid][2]) + (sh_grp[tid][1] + sh_grp[tid][3]);
        sh_r[tid] = 1.0f / sqrtf(total / 128.0f + prm.epsilon);
    }
    __syncthreads();
    // (3) One thread per (row, four rotate_half pairs) for the row's three vectors, which share the
    //     RoPE row (and the two q heads their gamma): normalise, gamma, RoPE with every bf16 rounding
    //     of R17:12207-12279.
    for (int it = tid; it < rows * 16; it += kPredThreads) {
        const int vrow = it >> 4, d0 = (it & 15) * 4;
        const uint2 cl = *reinterpret_cast<const uint2*>(&sh_cos[vrow][d0]), ch = *reinterpret_cast<const uint2*>(&sh_cos[vrow][d0 + 64]);
        const uint2 sl = *reinterpret_cast<const uint2*>(&sh_sin[vrow][d0]), sh2 = *reinterpret_cast<const uint2*>(&sh_sin[vrow][d0 + 64]);
        const uint32_t clw[2] = {cl.x, cl.y}, chw[2] = {ch.x, ch.y}, slw[2] = {sl.x, sl.y}, shw[2] = {sh2.x, sh2.y};
        float c0[4], c1[4], s0[4], s1[4];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            c0[2 * j] = lo_bf16(clw[j]); c0[2 * j + 1] = hi_bf16(clw[j]);
            c1[2 * j] = lo_bf16(chw[j]); c1[2 * j + 1] = hi_bf16(chw[j]);
            s0[2 * j] = lo_bf16(slw[j]); s0[2 * j + 1] = hi_bf16(slw[j]);
            s1[2 * j] = lo_bf16(shw[j]); s1[2 * j + 1] = hi_bf16(shw[j]);
        }
        float g0[4], g1[4];
#pragma unroll
        for (int which = 0; which < 3; ++which) {
            if (which != 1) {   // head 1 reuses head 0's gamma
                const uint16_t* gamma = sh_gamma[which < 2 ? 0 : 1];
                const uint2 gl = *reinterpret_cast<const uint2*>(gamma + d0), gh = *reinterpret_cast<const uint2*>(gamma + d0 + 64);
                g0[0] = lo_bf16(gl.x); g0[1] = hi_bf16(gl.x); g0[2] = lo_bf16(gl.y); g0[3] = hi_bf16(gl.y);
                g1[0] = lo_bf16(gh.x); g1[1] = hi_bf16(gh.x); g1[2] = lo_bf16(gh.y); g1[3] = hi_bf16(gh.y);
            }
            uint16_t* x = which < 2 ? sh_q[which][vrow] : sh_k[key_row_of(vrow)];
            const float r = sh_r[vrow * 3 + which];
            const uint2 xl = *reinterpret_cast<const uint2*>(x + d0), xh = *reinterpret_cast<const uint2*>(x + d0 + 64);
            const float x0[4] = {lo_bf16(xl.x), hi_bf16(xl.x), lo_bf16(xl.y), hi_bf16(xl.y)};
            const float x1[4] = {lo_bf16(xh.x), hi_bf16(xh.x), lo_bf16(xh.y), hi_bf16(xh.y)};
            float res_lo[4], res_hi[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float n0, n1, w0, w1, f0, f1, t0, t1;
                round_bf16_pair(x0[e] * r, x1[e] * r, n0, n1);
                round_bf16_pair(n0 * g0[e], n1 * g1[e], w0, w1);
                round_bf16_pair(w0 * c0[e], w1 * c1[e], f0, f1);
                round_bf16_pair((-w1) * s0[e], w0 * s1[e], t0, t1);
                res_lo[e] = f0 + t0;
                res_hi[e] = f1 + t1;
            }
            const uint32_t out_lo[2] = {pack_bf16_pair(res_lo[0], res_lo[1]), pack_bf16_pair(res_lo[2], res_lo[3])};
            const uint32_t out_hi[2] = {pack_bf16_pair(res_hi[0], res_hi[1]), pack_bf16_pair(res_hi[2], res_hi[3])};
            *reinterpret_cast<uint2*>(x + d0) = make_uint2(out_lo[0], out_lo[1]);
            *reinterpret_cast<uint2*>(x + d0 + 64) = make_uint2(out_hi[0], out_hi[1]);
            if (which == 2) {
                // every wave reads all of K for the scores: widen it once here instead of four times there
                *reinterpret_cast<float4*>(&sh_kf[key_row_of(vrow)][d0]) =
                    make_float4(lo_bf16(out_lo[0]), hi_bf16(out_lo[0]), lo_bf16(out_lo[1]), hi_bf16(out_lo[1]));
                *reinterpret_cast<float4*>(&sh_kf[key_row_of(vrow)][d0 + 64]) =
                    make_float4(lo_bf16(out_hi[0]), hi_bf16(out_hi[0]), lo_bf16(out_hi[1]), hi_bf16(out_hi[1]));
            }
        }
    }
    __syncthreads();

    }   // !STAGED

    // ---- optional K/V cache write-back, layout [unit][kv head][16][128] (R17:10711-10737) ---------
    if (APPEND) {
        if (tid < 32) {
            const int chunk = tid & 15, is_v = tid >> 4;
            *reinterpret_cast<uint4*>((is_v ? prm.v_cache_out : prm.k_cache_out)
                                      + (static_cast<int64_t>(kvh) * kPredRows + new_row) * kDim + chunk * 8) =
                *reinterpret_cast<const uint4*>(is_v ? &sh_v[new_row][chunk * 8] : &sh_k[new_row][chunk * 8]);
        }
    }
    if (MODE == 0 && prm.k_cache_out) {
        for (int c = tid; c < kPredRows * 16; c += kPredThreads) {
            const int row = c >> 4, chunk = c & 15;
            const int64_t dst = ((unit * 8 + kvh) * kPredRows + row) * kDim + chunk * 8;
            uint4 kv = make_uint4(0, 0, 0, 0), vv = make_uint4(0, 0, 0, 0);
            if (row < rows) {
                kv = *reinterpret_cast<const uint4*>(&sh_k[row][chunk * 8]);
                vv = *reinterpret_cast<const uint4*>(&sh_v[row][chunk * 8]);
            }
            *reinterpret_cast<uint4*>(prm.k_cache_out + dst) = kv;
            if (prm.v_cache_out) *reinterpret_cast<uint4*>(prm.v_cache_out + dst) = vv;
        }
    }

    // ---- scores ---------------------------------------------------------------------------------------
    // A 32-lane half wave evaluates one query vector against the keys 0..row in the reference's order
    // of operations (R17:12386-12418): reference lane v accumulates dims v, v+32, v+64, v+96 with fmaf,
    // then the shuffle tree (v + v^16, then ^8, ^4, ^2, ^1).  The tree runs as a reduce-scatter: at
    // every level a lane keeps half of its remaining keys and adds its partner's values for them,
    // which yields the same sums (fp addition is commutative) with 16 exchanges instead of 80; key j
    // ends in reference lanes 2j and 2j+1.  Physical lane p plays reference lane v(p), chosen so
    // that every partner is one cross-lane ALU operand away and nothing goes through LDS:
    // v = p with bits 1 and 0 flipped where bit 2 is set, which turns v^4 into the DPP
    // half-row mirror (p^7); v^16 is v_permlane16_swap, v^8 a DPP row rotation, v^2 and v^1 DPP quad
    // permutations.
    {
        const int half = lane >> 5;
        const int pl = lane & 31;
        const int hl = pl ^ ((pl & 4) ? 3 : 0);   // the reference lane this lane plays
        const float scale = __uint_as_float(0x3db504f3U);   // kAttentionScaleBits, R17:9354-9356
        float kf[kPredRows][4];
#pragma unroll
        for (int j = 0; j < kPredRows; ++j)
#pragma unroll
            for (int c = 0; c < 4; ++c) kf[j][c] = sh_kf[j][hl + 32 * c];
        auto dpp = [](float v, auto ctrl) {
            return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), decltype(ctrl)::value, 0xf, 0xf, false));
        };
        constexpr std::integral_constant<int, 0x128> kRowRor8{};        // lane p reads p ^ 8
        constexpr std::integral_constant<int, 0x141> kHalfMirror{};     // lane p reads p ^ 7
        constexpr std::integral_constant<int, 0x4e> kQuadXor2{};        // quad_perm [2,3,0,1]
        constexpr std::integral_constant<int, 0xb1> kQuadXor1{};        // quad_perm [1,0,3,2]
        // The two halves of a wave take the two heads of the same row, so that the keys after the
        // row (never read: the softmax masks them) are skipped with a wave-uniform branch.
        for (int row = wave; row < rows; row += 4) {
            const int g = half;
            float q4[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) q4[c] = bf2f(sh_q[g][row][hl + 32 * c]);
            float x[kPredRows];
#pragma unroll
            for (int j = 0; j < kPredRows; ++j) {
                float acc = 0.0f;
                if (j < limit_of(row)) {
                    asm volatile("" ::: "memory");   // keeps the branch: the compiler would compute and discard
#pragma unroll
                    for (int c = 0; c < 4; ++c) acc = fmaf(q4[c], kf[j][c], acc);
                }
                x[j] = acc;
            }
            // level 16: reference lanes 0..15 keep keys 0..7, lanes 16..31 keys 8..15.
            // v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even
            // rows of its second, so after swapping (x[j], x[j+8]) the two registers hold, in every
            // lane, its own and its partner's value of the key it keeps.
            float y8[8], y4[4], y2[2];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(x[j]), __float_as_uint(x[j + 8]), false, false);
                y8[j] = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
            }
            {
                const bool up = hl & 8;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float give = up ? y8[j] : y8[j + 4];
                    const float keep = up ? y8[j + 4] : y8[j];
                    y4[j] = keep + dpp(give, kRowRor8);
                }
            }
            {
                const bool up = hl & 4;
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const float give = up ? y4[j] : y4[j + 2];
                    const float keep = up ? y4[j + 2] : y4[j];
                    y2[j] = keep + dpp(give, kHalfMirror);
                }
            }
            float y1;
            {
                const bool up = hl & 2;
                const float give = up ? y2[0] : y2[1];
                const float keep = up ? y2[1] : y2[0];
                y1 = keep + dpp(give, kQuadXor2);
            }
            const float total = y1 + dpp(y1, kQuadXor1);
            if ((hl & 1) == 0) {
                const float raw = rbf(total);
                sh_s[g][row][hl >> 1] = rbf(raw * scale);
            }
        }
    }
    __syncthreads();

    // ---- softmax: one thread per (head, row) ----------------------------------------------------------
    // (an element-per-thread layout recomputes the row maximum and the row sum sixteen times; the
    // kernel is bound by VALU issue, so the 32 busy lanes of one wave are the cheaper choice)
    if (tid < 2 * rows) {
        const int g = tid / rows;
        const int r = tid % rows;
        const int limit = limit_of(r);
        float sc[kPredRows];
#pragma unroll
        for (int t = 0; t < kPredRows; t += 4) {
            const float4 v4 = *reinterpret_cast<const float4*>(&sh_s[g][r][t]);
            sc[t] = v4.x; sc[t + 1] = v4.y; sc[t + 2] = v4.z; sc[t + 3] = v4.w;
        }
        // maximum = maximum > s ? maximum : s over keys 0..r (R17:12449-12470); a masked key enters
        // as -inf, which never replaces anything
        float maximum = -INFINITY;
#pragma unroll
        for (int t = 0; t < kPredRows; ++t) {
            const float cand = t < limit ? sc[t] : -INFINITY;
            maximum = maximum > cand ? maximum : cand;
        }
        float e[kPredRows];
#pragma unroll
        for (int t = 0; t < kPredRows; ++t) e[t] = t < limit ? expf(sc[t] - maximum) : 0.0f;
        // exp() >= +0 and masked entries are +0: the full 16-leaf tree equals the reference's sum
        const float total = TreeSum<16, 0, 1>::eval([&](int t) { return e[t]; });
#pragma unroll
        for (int t = 0; t < kPredRows; t += 4) {
            float4 p4;
            p4.x = t < limit ? rbf(e[t] / total) : 0.0f;
            p4.y = t + 1 < limit ? rbf(e[t + 1] / total) : 0.0f;
            p4.z = t + 2 < limit ? rbf(e[t + 2] / total) : 0.0f;
            p4.w = t + 3 < limit ? rbf(e[t + 3] / total) : 0.0f;
            *reinterpret_cast<float4*>(&sh_s[g][r][t]) = p4;
        }
    }
    __syncthreads();

    // ---- P.V: thread (g, d) owns one output column for all rows -------------------------------------
    {
        const int g = tid >> 7;
        const int d = tid & 127;
        float vcol[kPredRows];
#pragma unroll
        for (int j = 0; j < kPredRows; ++j) vcol[j] = bf2f(sh_v[j][d]);
        uint16_t* out = prm.out + ((unit * rows) * 16 + kvh * 2 + g) * kDim + d;
        if (STAGED || APPEND) {
            for (int r = 0; r < rows; ++r)
                out[r * 16 * kDim] = __builtin_bit_cast(uint16_t, static_cast<__bf16>(pv_limited(sh_s[g][r], vcol, limit_of(r))));
        } else {
            pv_rows<0>(sh_s[g], vcol, out, 16 * kDim, rows);
        }
    }
}

}  // namespace qm

extern "C" int32_t qm_predictor_attention_loop(
    const uint16_t* q, const uint16_t* k, const uint16_t* v,
    const uint16_t* q_norm_w, const uint16_t* k_norm_w,
    const uint16_t* cos_rows, const uint16_t* sin_rows,
    uint16_t* context_out, uint16_t* k_cache_out, uint16_t* v_cache_out,
    int32_t units, int32_t n_layers, int32_t rows, int32_t first_rows,
    float epsilon, void* hip_stream) {
    if (!q || !k || !v || !q_norm_w || !k_norm_w || !cos_rows || !sin_rows || !context_out)
        return QM_ERR_NULL;
    if (units < 0 || units > 65535 * 64 || n_layers <= 0 || rows < 1 || rows > qm::kPredRows)
        return QM_ERR_ARGUMENT;
    // first_rows = 2 is the reference's two-row causal step 0 (R17:13593-13596); it renumbers
    // the steps but row r still attends keys 0..r, so both values run the same kernel.
    if ((first_rows != 1 && first_rows != 2) || first_rows > rows) return QM_ERR_ARGUMENT;
    if (v_cache_out && !k_cache_out) return QM_ERR_ARGUMENT;
    const uintptr_t align = reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k)
                          | reinterpret_cast<uintptr_t>(v) | reinterpret_cast<uintptr_t>(k_cache_out)
                          | reinterpret_cast<uintptr_t>(v_cache_out);
    if (align & 15) return QM_ERR_GEOMETRY;
    if (units == 0) return QM_OK;
    const int32_t kernel = qm::option_value(QM_OPT_PREDICTOR_LOOP_KERNEL);
    if (kernel < 0 || kernel > 1) return QM_ERR_ARGUMENT;
    qm::PredictorParams prm;
    prm.q = q; prm.k = k; prm.v = v;
    prm.q_norm_w = q_norm_w; prm.k_norm_w = k_norm_w;
    prm.cos_rows = cos_rows; prm.sin_rows = sin_rows;
    prm.out = context_out; prm.k_cache_out = k_cache_out; prm.v_cache_out = v_cache_out;
    prm.unit_base = 0; prm.n_layers = n_layers; prm.rows = rows; prm.epsilon = epsilon;
    prm.key_length = 0; prm.causal = 1;
    if (kernel == 0) {
        const uintptr_t more = reinterpret_cast<uintptr_t>(q_norm_w) | reinterpret_cast<uintptr_t>(k_norm_w)
                             | reinterpret_cast<uintptr_t>(cos_rows) | reinterpret_cast<uintptr_t>(sin_rows);
        if (more & 15) return QM_ERR_GEOMETRY;
        return qm::launch_predictor_loop_mfma(prm, units, static_cast<hipStream_t>(hip_stream));
    }
    // grid.y is limited to 65535: fold large unit counts into several launches.
    const int32_t per_launch = 65535;
    for (int32_t first = 0; first < units; first += per_launch) {
        const int32_t n = units - first < per_launch ? units - first : per_launch;
        qm::PredictorParams p = prm;
        const int64_t row0 = static_cast<int64_t>(first) * rows;
        p.q = q + row0 * 16 * qm::kDim;
        p.k = k + row0 * 8 * qm::kDim;
        p.v = v + row0 * 8 * qm::kDim;
        p.out = context_out + row0 * 16 * qm::kDim;
        if (k_cache_out) p.k_cache_out = k_cache_out + static_cast<int64_t>(first) * 8 * 16 * qm::kDim;
        if (v_cache_out) p.v_cache_out = v_cache_out + static_cast<int64_t>(first) * 8 * 16 * qm::kDim;
        p.unit_base = first;
        hipLaunchKernelGGL(qm::predictor_loop_kernel<0>, dim3(8, n), dim3(qm::kPredThreads), 0,
                           static_cast<hipStream_t>(hip_stream), p);
        const int32_t rc = qm::launch_status();
        if (rc != QM_OK) return rc;
    }
    return QM_OK;
}

extern "C" int32_t qm_predictor_attention_staged(const uint16_t* query_bhsd, const uint16_t* key_cache,
                                                 const uint16_t* value_cache, uint16_t* output, int32_t rows,
                                                 int32_t key_length, int32_t causal_prefill, void* hip_stream) {
    if (!query_bhsd || !key_cache || !value_cache || !output) return QM_ERR_NULL;
    if (rows < 1 || rows > qm::kPredRows || key_length < 1 || key_length > qm::kPredRows) return QM_ERR_ARGUMENT;
    const uintptr_t align = reinterpret_cast<uintptr_t>(query_bhsd) | reinterpret_cast<uintptr_t>(key_cache)
                          | reinterpret_cast<uintptr_t>(value_cache);
    if (align & 15) return QM_ERR_GEOMETRY;
    qm::PredictorParams prm = {};
    prm.q = query_bhsd; prm.k = key_cache; prm.v = value_cache;
    prm.out = output;
    prm.unit_base = 0; prm.n_layers = 1; prm.rows = rows; prm.epsilon = 0.0f;
    prm.key_length = key_length; prm.causal = causal_prefill ? 1 : 0;
    hipLaunchKernelGGL(qm::predictor_loop_kernel<1>, dim3(8, 1), dim3(qm::kPredThreads), 0,
                       static_cast<hipStream_t>(hip_stream), prm);
    return qm::launch_status();
}

extern "C" int32_t qm_predictor_step_attention_m1(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                                                  const uint16_t* q_norm_w, const uint16_t* k_norm_w,
                                                  const uint16_t* cos_row, const uint16_t* sin_row,
                                                  uint16_t* key_cache, uint16_t* value_cache, uint16_t* context_out,
                                                  int32_t cache_position, float epsilon, void* hip_stream) {
    if (!q || !k || !v || !q_norm_w || !k_norm_w || !cos_row || !sin_row || !key_cache || !value_cache || !context_out)
        return QM_ERR_NULL;
    if (cache_position < 0 || cache_position >= qm::kPredRows) return QM_ERR_SLOT_RANGE;
    const uintptr_t align = reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v)
                          | reinterpret_cast<uintptr_t>(q_norm_w) | reinterpret_cast<uintptr_t>(k_norm_w)
                          | reinterpret_cast<uintptr_t>(cos_row) | reinterpret_cast<uintptr_t>(sin_row)
                          | reinterpret_cast<uintptr_t>(key_cache) | reinterpret_cast<uintptr_t>(value_cache);
    if (align & 15) return QM_ERR_GEOMETRY;
    qm::PredictorParams prm = {};
    prm.q = q; prm.k = k; prm.v = v;
    prm.q_norm_w = q_norm_w; prm.k_norm_w = k_norm_w;
    prm.cos_rows = cos_row; prm.sin_rows = sin_row;
    prm.out = context_out; prm.k_cache_out = key_cache; prm.v_cache_out = value_cache;
    prm.unit_base = 0; prm.n_layers = 1; prm.rows = 1; prm.epsilon = epsilon;
    prm.key_length = cache_position + 1; prm.causal = 0;
    hipLaunchKernelGGL(qm::predictor_loop_kernel<2>, dim3(8, 1), dim3(qm::kPredThreads), 0,
                       static_cast<hipStream_t>(hip_stream), prm);
    return qm::launch_status();
}
