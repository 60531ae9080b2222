// qm_predictor_mfma.hip — the code predictor's per-frame attention loop on the matrix cores (gfx950).
//
// One 64-lane wave owns one (unit, kv head) item, unit = (frame, layer), start to end; the four waves of
// a block share only the RoPE rows and norm weights, staged once in LDS.  Q (two heads), K and the RoPE rows are loaded straight into the
// MFMA operand layout of v_mfma_f32_16x16x32_bf16 — lane l holds vector (row) l % 16, dimensions
// 32 kb + 8 (l / 16) + e, kb = 0..3, e = 0..7 — in which
//   * the reference's 32-dimension groups of the sum of squares are the four kb register sets, and
//     its 32-lane shuffle tree (R17:8233-8245) pairs elements through two lane exchanges
//     (v_permlane32_swap, v_permlane16_swap) and three in-register levels, evaluated as a
//     reduce-scatter: same pairs, same order of fp32 additions, same bits;
//   * the rotate_half partner of dimension d is d + 64 = register set kb + 2 of the same lane.
// QK-RMSNorm + RoPE therefore keep every bf16 rounding and the summation order of R17:12133-12307:
// the rotated K (and the cache write-back) are bit-identical to the exact-chain kernel.
// Scores S^T = K Q^T are four 16x16x32 MFMAs per head, rounded bf16(QK), bf16(* scale) like the
// reference (R17:12409-12418); the softmax of a row runs in fp32 over the accumulator layout
// (lane l: query row l % 16, keys 4 (l / 16) + i), P is rounded to bf16 like the reference
// (R17:12500-12507) and is, in that layout, the B operand of O^T += V^T P^T with
// v_mfma_f32_16x16x16_bf16; V^T fragments come from a 4 KiB LDS tile through the transposing read
// ds_read_b64_tr_b16.  What differs from the exact-chain kernel: fp32 sums inside the two
// products are the matrix core's, the exponential is v_exp_f32 and the division a reciprocal —
// within the operator's tolerance (max abs error <= 1e-2), not bit-identical.
//
// Per item: 16 KiB in, 8 KiB out (+ 8 KiB with the cache write-back); about 1 700 vector
// instructions against 7 000 of the exact-chain kernel, which is bound by VALU issue.  The context
// rows are staged through the (consumed) V tile so that global stores are 16 bytes per lane:
// 8-byte stores straight from the accumulator layout cost 59 us instead of 50 us at 256 x 5 x 16.
// Non-temporal loads and stores were measured and are slower here (52 us).

#include "qm_device.h"
#include "qm_host.h"
#include "qm_predictor_params.h"

namespace qm {

namespace {

typedef short s16x4_t __attribute__((ext_vector_type(4)));

constexpr int kVRowBytes = 272;                    // LDS row of the V tile: 256 B + 16 B of padding
constexpr int kVTileBytes = kPredRows * kVRowBytes;

__device__ __forceinline__ float swap32_add(float a, float b) {
    // lanes 0..31: a[l] + a[l + 32]; lanes 32..63: b[l - 32] + b[l]
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float swap16_add(float a, float b) {
    // 16-lane rows [a0 + a1, b0 + b1, a2 + a3, b2 + b3]
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float swap32_max(float a) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(a), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float swap16_max(float a) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(a), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// The 128 values of a head vector as this lane holds them: set kb, element e = dimension 32 kb + 8 G + e.
struct VecRegs {
    uint4 raw[4];
};

__device__ __forceinline__ float elem(const VecRegs& v, int kb, int e) {
    const uint32_t w = e < 2 ? v.raw[kb].x : e < 4 ? v.raw[kb].y : e < 6 ? v.raw[kb].z : v.raw[kb].w;
    return (e & 1) ? hi_bf16(w) : lo_bf16(w);
}

// Sum of squares of the vector (l % 16) in every lane, in the reference's order (R17:8233-8271):
// inside each 32-dimension group the tree x[i] + x[i + 16], then + 8, + 4, + 2, + 1 with
// i = 8 (l / 16) + e; then (w0 + w2) + (w1 + w3) over the four groups.
__device__ __forceinline__ float vector_sum_squares(const VecRegs& v) {
    float u[4];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
        float sq[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float x = elem(v, kb, e);
            sq[e] = x * x;
        }
        // level 16: lanes l and l + 32.  Lower half keeps elements 0..3, upper half 4..7.
        float c[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) c[e] = swap32_add(sq[e], sq[e + 4]);
        // level 8: lanes l and l + 16.  Rows then hold elements [e, e + 2, e + 4, e + 6].
        const float d0 = swap16_add(c[0], c[2]);
        const float d1 = swap16_add(c[1], c[3]);
        // level 4: element x with x + 4 = rows 0 with 2, 1 with 3.  Rows: [U0, U2, U1, U3].
        u[kb] = swap32_add(d0, d1);
    }
    // level 2 (U0 + U2, U1 + U3) for two groups at a time: rows [W0 a, W0 b, W1 a, W1 b]
    const float x01 = swap16_add(u[0], u[1]);
    const float x23 = swap16_add(u[2], u[3]);
    // level 1 (W0 + W1): rows [w0, w1, w2, w3], the four group sums
    const float w = swap32_add(x01, x23);
    // (w0 + w2) + (w1 + w3)
    const float y = swap32_add(w, w);       // rows [w0 + w2, w1 + w3, w0 + w2, w1 + w3]
    return swap16_add(y, y);
}

// One register set of an operand row kept in LDS: dimensions 32 kb + 8 G .. + 7 of `row` (16 bytes).
__device__ __forceinline__ uint4 lds_set(const unsigned char* row, int kb, int grp) {
    return *reinterpret_cast<const uint4*>(row + 64 * kb + 16 * grp);
}
// a.lo * b.lo + a.hi * b.hi of packed bf16 pairs, two or four at a time, in the three-operand encoding with
// a literal 0 addend (the compiler's own choice, the two-operand form, needs a zeroed accumulator register
// per use).  The compiler cannot see through an assembly statement, so the wait states this chip wants
// between a dot-product instruction's write and another instruction's read of it (three) are part of the
// statement: the results of a group are independent of one another and one s_nop ends the group.
__device__ __forceinline__ void dot2_pairs_x2(uint32_t a0, uint32_t b0, uint32_t a1, uint32_t b1, float& d0, float& d1) {
    asm("v_dot2_f32_bf16 %0, %2, %3, 0\n\tv_dot2_f32_bf16 %1, %4, %5, 0\n\ts_nop 2"
        : "=&v"(d0), "=&v"(d1) : "v"(a0), "v"(b0), "v"(a1), "v"(b1));
}
__device__ __forceinline__ void dot2_pairs_x4(uint32_t a0, uint32_t b0, uint32_t a1, uint32_t b1, uint32_t a2, uint32_t b2,
                                              uint32_t a3, uint32_t b3, float& d0, float& d1, float& d2, float& d3) {
    asm("v_dot2_f32_bf16 %0, %4, %5, 0\n\tv_dot2_f32_bf16 %1, %6, %7, 0\n\t"
        "v_dot2_f32_bf16 %2, %8, %9, 0\n\tv_dot2_f32_bf16 %3, %10, %11, 0\n\ts_nop 2"
        : "=&v"(d0), "=&v"(d1), "=&v"(d2), "=&v"(d3)
        : "v"(a0), "v"(b0), "v"(a1), "v"(b1), "v"(a2), "v"(b2), "v"(a3), "v"(b3));
}

__device__ __forceinline__ uint32_t word_of(const uint4& raw, int e) {
    return e < 2 ? raw.x : e < 4 ? raw.y : e < 6 ? raw.z : raw.w;
}

// bf16(value) placed in the half of a packed pair that element e occupies (even e: low), the other half +0.
__device__ __forceinline__ uint32_t round_into_slot(float value, int e) {
    return (e & 1) ? pack_bf16_pair(0.0f, value) : pack_bf16_pair(value, 0.0f);
}

// RMSNorm + RoPE of the vector in place (packed bf16), every rounding of R17:12207-12279.
// gamma, cosv, sinv: LDS rows of 128 bf16 (the norm weight; the RoPE row of this lane's vector).
// A product of two bf16 values is exact in fp32, so bf16(a) * b is taken as
// v_dot2_f32_bf16((bf16(a), 0), (b, neighbour)) straight from the packed operands: nothing is
// unpacked, and the rounding instruction is the conversion itself.  The last step,
// bf16(w cos) + bf16(rotated w sin), is the same instruction on (1, +-1).  (A product that is an
// exact zero may come out as +0 where a scalar multiply gives -0.)
__device__ __forceinline__ void norm_rope_vector(VecRegs& v, const unsigned char* gamma, const unsigned char* cosv,
                                                 const unsigned char* sinv, float epsilon, int grp) {
    const float total = vector_sum_squares(v);
    const float r = 1.0f / sqrtf(total / 128.0f + epsilon);
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
        const uint4 g0 = lds_set(gamma, kb, grp), g1 = lds_set(gamma, kb + 2, grp);
        const uint4 c0 = lds_set(cosv, kb, grp), c1 = lds_set(cosv, kb + 2, grp);
        const uint4 s0 = lds_set(sinv, kb, grp), s1 = lds_set(sinv, kb + 2, grp);
        float lo[8], hi[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float x0 = elem(v, kb, e), x1 = elem(v, kb + 2, e);
            const uint32_t n0 = round_into_slot(x0 * r, e), n1 = round_into_slot(x1 * r, e);
            float g_0, g_1, f0, f1, t0, t1;
            dot2_pairs_x2(n0, word_of(g0, e), n1, word_of(g1, e), g_0, g_1);
            const uint32_t w0 = round_into_slot(g_0, e), w1 = round_into_slot(g_1, e);
            dot2_pairs_x4(w0, word_of(c0, e), w1, word_of(c1, e), w1, word_of(s0, e), w0, word_of(s1, e), f0, f1, t0, t1);
            // dimension d < 64: bf16(w0 cos) + bf16(-w1 sin) = bf16(w0 cos) - bf16(w1 sin); d + 64: both added
            dot2_pairs_x2(pack_bf16_pair(f0, t0), 0xBF803F80U, pack_bf16_pair(f1, t1), 0x3F803F80U, lo[e], hi[e]);
        }
        v.raw[kb] = make_uint4(pack_bf16_pair(lo[0], lo[1]), pack_bf16_pair(lo[2], lo[3]),
                               pack_bf16_pair(lo[4], lo[5]), pack_bf16_pair(lo[6], lo[7]));
        v.raw[kb + 2] = make_uint4(pack_bf16_pair(hi[0], hi[1]), pack_bf16_pair(hi[2], hi[3]),
                                   pack_bf16_pair(hi[4], hi[5]), pack_bf16_pair(hi[6], hi[7]));
    }
}

__device__ __forceinline__ VecRegs load_vector(const uint16_t* base, bool valid) {
    VecRegs v;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
        v.raw[kb] = make_uint4(0, 0, 0, 0);
        if (valid) v.raw[kb] = *reinterpret_cast<const uint4*>(base + 32 * kb);
    }
    return v;
}

}  // namespace

// grid: ceil(units * 8 / 4) blocks of 256 threads; wave w of block b owns item 4 b + w,
// item = unit * 8 + kv head.
__global__ __launch_bounds__(kPredThreads, 4) void predictor_loop_mfma_kernel(PredictorParams prm, int64_t items) {
    request_arguments(prm, items);
    __shared__ __attribute__((aligned(16))) unsigned char sh_v[4][kVTileBytes];
    __shared__ __attribute__((aligned(16))) unsigned char sh_cos[kVTileBytes];      // [row][128] bf16, padded rows
    __shared__ __attribute__((aligned(16))) unsigned char sh_sin[kVTileBytes];
    __shared__ __attribute__((aligned(16))) unsigned char sh_gamma[2][256];         // q, k norm weights

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int64_t item_raw = static_cast<int64_t>(blockIdx.x) * 4 + wave;
    const bool has_item = item_raw < items;
    const int64_t item = has_item ? item_raw : items - 1;
    const int64_t unit = item >> 3;
    const int kvh = static_cast<int>(item & 7);
    const int rows = prm.rows;
    // the four items of a block are four kv heads of one unit: one layer, one pair of norm weights
    const int layer = static_cast<int>((prm.unit_base + (static_cast<int64_t>(blockIdx.x) >> 1)) % prm.n_layers);
    const int vec = lane & 15;            // the row (token) this lane's vectors belong to
    const int grp = lane >> 4;            // G: dimensions 8 G .. 8 G + 7 of every 32
    const bool valid = vec < rows;
    const int64_t row64 = unit * rows + vec;
    const int dim0 = 8 * grp;

    // ---- the item's own loads are requested first; the block's shared operands go through LDS ----
    const VecRegs vv = load_vector(prm.v + (row64 * 8 + kvh) * kDim + dim0, valid);
    VecRegs kk = load_vector(prm.k + (row64 * 8 + kvh) * kDim + dim0, valid);
    VecRegs q0 = load_vector(prm.q + (row64 * 16 + 2 * kvh) * kDim + dim0, valid);
    VecRegs q1 = load_vector(prm.q + (row64 * 16 + 2 * kvh + 1) * kDim + dim0, valid);
    {
        // RoPE rows: 16 x 256 B each, thread t moves piece t % 16 of row t / 16; norm weights: 2 x 256 B
        const int srow = tid >> 4, piece = tid & 15;
        uint4 c = make_uint4(0, 0, 0, 0), sn = make_uint4(0, 0, 0, 0);
        if (srow < rows) {
            c = *reinterpret_cast<const uint4*>(prm.cos_rows + srow * kDim + 8 * piece);
            sn = *reinterpret_cast<const uint4*>(prm.sin_rows + srow * kDim + 8 * piece);
        }
        *reinterpret_cast<uint4*>(sh_cos + srow * kVRowBytes + 16 * piece) = c;
        *reinterpret_cast<uint4*>(sh_sin + srow * kVRowBytes + 16 * piece) = sn;
        if (tid < 32) {
            const uint16_t* w = (tid < 16 ? prm.q_norm_w : prm.k_norm_w) + layer * kDim + 8 * piece;
            *reinterpret_cast<uint4*>(sh_gamma[tid >> 4] + 16 * piece) = *reinterpret_cast<const uint4*>(w);
        }
    }
    __syncthreads();
    if (!has_item) return;

    // ---- QK-RMSNorm + RoPE, one vector after the other (the fences keep the compiler from interleaving
    // them, which triples the registers) ----
    const unsigned char* my_cos = sh_cos + vec * kVRowBytes;
    const unsigned char* my_sin = sh_sin + vec * kVRowBytes;
    norm_rope_vector(kk, sh_gamma[1], my_cos, my_sin, prm.epsilon, grp);
    __builtin_amdgcn_sched_barrier(0);
    norm_rope_vector(q0, sh_gamma[0], my_cos, my_sin, prm.epsilon, grp);
    __builtin_amdgcn_sched_barrier(0);
    norm_rope_vector(q1, sh_gamma[0], my_cos, my_sin, prm.epsilon, grp);
    __builtin_amdgcn_sched_barrier(0);
    if (!valid) {
        // rows beyond `rows` are never attended (causal) and are written back as zeros
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) kk.raw[kb] = q0.raw[kb] = q1.raw[kb] = make_uint4(0, 0, 0, 0);
    }

    // ---- V tile to LDS (row-major, padded rows), optional cache write-back [unit][kv head][16][128] ----
    unsigned char* vt = sh_v[wave];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
        *reinterpret_cast<uint4*>(vt + vec * kVRowBytes + 2 * (32 * kb + dim0)) = vv.raw[kb];
    if (prm.k_cache_out) {
        const int64_t dst = ((unit * 8 + kvh) * kPredRows + vec) * kDim + dim0;
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) {
            *reinterpret_cast<uint4*>(prm.k_cache_out + dst + 32 * kb) = kk.raw[kb];
            if (prm.v_cache_out) *reinterpret_cast<uint4*>(prm.v_cache_out + dst + 32 * kb) = vv.raw[kb];
        }
    }

    // ---- scores: S^T[key][query row] per head, keys on MFMA rows ----
    f32x4_t s0 = {0.0f, 0.0f, 0.0f, 0.0f}, s1 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
        const bf16x8_t kf = __builtin_bit_cast(bf16x8_t, kk.raw[kb]);
        s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, __builtin_bit_cast(bf16x8_t, q0.raw[kb]), s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, __builtin_bit_cast(bf16x8_t, q1.raw[kb]), s1, 0, 0, 0);
    }

    // ---- softmax of query row `vec` over keys 4 G + i <= vec, both heads; P as bf16 ----
    const float scale = __uint_as_float(0x3db504f3U);   // kAttentionScaleBits, R17:9354-9356
    s16x4_t p[2];
#pragma unroll
    for (int g = 0; g < 2; ++g) {
        const f32x4_t s = g == 0 ? s0 : s1;
        float sc[4];
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float raw = round_bf16(s[i]);
            sc[i] = 4 * grp + i <= vec ? round_bf16(raw * scale) : -INFINITY;
            mx = fmaxf(mx, sc[i]);
        }
        mx = swap32_max(swap16_max(mx));               // key 0 is never masked: finite
        float e[4], sum = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            e[i] = fast_exp2((sc[i] - mx) * kLog2e);
            sum += e[i];
        }
        sum = swap16_add(sum, sum);
        sum = swap32_add(sum, sum);
        const float inv = __builtin_amdgcn_rcpf(sum);
        const uint32_t lo = pack_bf16_pair(e[0] * inv, e[1] * inv);
        const uint32_t hi = pack_bf16_pair(e[2] * inv, e[3] * inv);
        p[g] = __builtin_bit_cast(s16x4_t, make_uint2(lo, hi));
    }

    // ---- O^T += V^T P^T: eight 16-dimension tiles, V^T fragments by transposing reads ----
    // One ds_read_b64_tr_b16 of 16 lanes takes a block of 4 keys x 16 dimensions (lane 4 j + c of the
    // 16 addresses dimensions 4 c .. 4 c + 3 of key j) and gives lane i the four keys of dimension i:
    // lane group G reads keys 4 G .. 4 G + 3, the k indices of its MFMA operand.
    const uint32_t v_lds = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) unsigned char*)vt))
                         + (4 * grp + ((lane >> 2) & 3)) * kVRowBytes + 8 * (lane & 3);
    __builtin_amdgcn_s_waitcnt(0xc07f);               // lgkmcnt(0): this wave's own LDS writes have landed
    __builtin_amdgcn_wave_barrier();
    unsigned long long frag[8];
#pragma unroll
    for (int t = 0; t < 8; ++t)
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(frag[t]) : "v"(v_lds), "n"(32 * t) : "memory");
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(frag[0]), "+v"(frag[1]), "+v"(frag[2]), "+v"(frag[3]), "+v"(frag[4]), "+v"(frag[5]), "+v"(frag[6]), "+v"(frag[7])
                 :
                 : "memory");
    __builtin_amdgcn_wave_barrier();
    // The V tile has been read: its LDS rows now stage one head's context at a time ([row][128] bf16), so that
    // the global stores are 16 bytes per lane, 256 contiguous bytes per row.
#pragma unroll
    for (int g = 0; g < 2; ++g) {
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            f32x4_t o = {0.0f, 0.0f, 0.0f, 0.0f};
            o = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4_t, frag[t]), p[g], o, 0, 0, 0);
            // lane: query row `vec`, dimensions 16 t + 4 G + 0..3
            *reinterpret_cast<uint2*>(vt + vec * kVRowBytes + 2 * (16 * t + 4 * grp)) =
                make_uint2(pack_bf16_pair(o[0], o[1]), pack_bf16_pair(o[2], o[3]));
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int orow = 4 * j + grp;             // 16 lanes move one row: piece `vec` of row orow
            const uint4 val = *reinterpret_cast<const uint4*>(vt + orow * kVRowBytes + 16 * vec);
            if (orow < rows)
                *reinterpret_cast<uint4*>(prm.out + ((unit * rows + orow) * 16 + 2 * kvh + g) * kDim + 8 * vec) = val;
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);           // the rows have been read before the next head overwrites them
        __builtin_amdgcn_wave_barrier();
    }
}

int32_t launch_predictor_loop_mfma(const PredictorParams& prm, int64_t units, hipStream_t stream) {
    const int64_t items = units * 8;
    const int64_t blocks = (items + 3) / 4;
    if (blocks > 0x7fffffffLL) return QM_ERR_ARGUMENT;
    hipLaunchKernelGGL(predictor_loop_mfma_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kPredThreads), 0, stream,
                       prm, items);
    return launch_status();
}

}  // namespace qm
