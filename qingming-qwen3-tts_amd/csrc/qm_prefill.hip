// qm_prefill.hip — causal GQA prefill attention on gfx950 bf16 MFMA, fused with the paged K/V write.
//
// Tiling.  A block of four waves owns 64 query rows of one (batch, kv head) and both query heads
// of the GQA pair: a wave's MFMA column dimension is 32 = 16 rows x 2 heads, so every K and V
// fragment read from LDS feeds both heads.  Keys are streamed in tiles of 64 through two LDS
// stages (global loads for the next tile are in flight while the current one is multiplied).
// A wave computes S^T = K Q^T with v_mfma_f32_32x32x16_bf16 (keys on MFMA rows, query columns on
// lanes), so that the softmax statistics of a query column live in one lane pair, and the
// accumulator layout of S^T is directly the B-operand layout of O^T += V^T P^T.  V is transposed
// on its way into LDS ([dim][key slot], key slots permuted to match the accumulator layout,
// 8-slot blocks XOR-swizzled per 16 rows so both the transposing writes and the fragment reads
// are conflict-free).
//
// Occupancy and what bounds the kernel.  A wave cannot issue VALU work in the shadow of its own
// MFMAs (measured: one MFMA plus eight independent FMAs take the sum of both), so the matrix pipe
// and the VALU only overlap between waves, and with two waves per SIMD whose phases are long (eight
// MFMAs, then about 150 VALU instructions, then eight MFMAs) that overlap is small as well: a
// synthetic pair of such waves takes 2 045 cycles per step against 2 420 serial and 1 216 ideal.
// The kernel therefore stays within 256 registers and 72 KB of LDS so that two blocks share a CU
// and fill each other's waits, and otherwise keeps the instruction count per key tile low.
// Variants that were measured and dropped (batch 4 x 1024 tokens / 4 x 4096 tokens, this one:
// 42 us / 381 us): a software pipeline inside the wave with three LDS stages and 316 registers,
// one wave per SIMD (51 us / 467 us); eight-wave blocks whose two wave groups split each key tile
// and merge through LDS, with phase-skewed groups and each block taking a heavy and a light
// query tile (41 us / 421 us: the longest block is halved, but the groups meet at a barrier per
// tile and run in step).  At batch 4 x 1024 tokens the time is the serial length of the blocks
// that own the last query tiles (16 key tiles at 1.7 us) plus a 4 us start in which every block
// fetches its first tiles from HBM at once, not chip throughput.
//
// Lazy rescale.  The running maximum of a column is only raised when a chunk exceeds it by more
// than kRescaleSlack (then O and the running sum are rescaled); otherwise probabilities are taken
// relative to the slightly stale maximum and may reach e^slack, which bf16 P and the fp32
// accumulators hold without loss of relative precision.
//
// Scheduling.  Blocks are numbered heaviest query tile first; the hardware hands the next
// (lighter) block to whichever CU retires one.  Blocks that share K/V differ by a multiple of
// batch*kv_heads and therefore land on the same XCD and hit its L2.
//
// Rounding.  With score rounding on (the default) scores are rounded to bf16 before and after
// scaling like the reference (R17:15879-15890); with it off they stay fp32 (8 VALU instructions
// fewer per score pair).  Softmax runs online in fp32; P enters the P.V MFMA as bf16 and the running
// sum adds the same rounded values — except in the first query tile, whose rows have so few keys
// that outputs are large: there P is split into hi + lo bf16 parts (two MFMAs) to stay inside the
// 1e-2 output tolerance.
//
// Causality.  A key after a query row never contributes; keys of later 16-row groups are not
// read into the product at all.  Inside a wave's own 16-row diagonal group the mask is P = 0
// times V, so a non-finite V of a later row of the same group would propagate (the reference
// skips those keys; finite values, the only ones a prefill produces, behave identically).
//
// Algorithmic work per (batch, kv head): flops = 2 heads * 2 matmuls * 2 * 128 * S(S+1)/2;
// HBM bytes = Q + O (2 heads) + K + V read once + K + V written to pages.  Bound: MFMA (with the
// softmax VALU work — 16 exponentials and two bf16 roundings per lane per 32 keys — as the
// practical limiter).

#include "qm_device.h"
#include "qm_host.h"

#include <type_traits>

namespace qm {

constexpr int kPfThreads = 256;
constexpr int kPfStages = 2;
constexpr int kBM = 64;          // query rows per block
constexpr int kBN = 64;          // keys per tile
constexpr int kKS = kDim + 8;    // LDS row stride of the K tile (elements)
constexpr int kVS = kBN + 8;     // LDS row stride of the V^T tile (elements)
constexpr int kOS = kDim + 8;    // LDS row stride of the output staging tile
constexpr float kRescaleSlack = 6.0f;

typedef float f32x16_t __attribute__((ext_vector_type(16)));

struct PrefillParams {
    const uint16_t* q;     // [batch][seq][2*kv_heads][128]
    const uint16_t* k;     // [batch][seq][kv_heads][128]
    const uint16_t* v;
    uint16_t* out;         // [batch][seq][2*kv_heads][128]
    const int32_t* page_table;   // [batch][max_pages] or NULL
    uint32_t* status;
    int64_t kv_stride_token;     // elements between consecutive keys of one kv head
    int64_t kv_stride_head;
    int64_t kv_stride_batch;
    PageMap pages;
    int has_cache;
    int batch;
    int seq;
    int kv_heads;
    int n_qtiles;
    float scale;
};

struct PfStage {
    uint16_t k[kBN * kKS];
    uint16_t vt[kDim * kVS];
};

// P of one 32-key chunk as MFMA B operands: two 16-key groups; lo only in the split-precision path.
struct PFrag {
    bf16x8_t hi[2];
    bf16x8_t lo[2];
};

// LDS slot of key j (0..15) inside a 16-key group: MFMA k index 8*g + e holds the key that the
// S^T accumulator register e of lane group g belongs to.
__device__ __forceinline__ int key_slot(int j) {
    return 8 * ((j & 7) >> 2) + 4 * (j >> 3) + (j & 3);
}

__device__ __forceinline__ bf16x8_t lds_frag(const uint16_t* p) {
    return *reinterpret_cast<const bf16x8_t*>(p);
}

// Both 32-lane halves receive max / sum over the two halves (v_permlane32_swap).
__device__ __forceinline__ float halves_max(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float halves_sum(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

template <int N> using int_c = std::integral_constant<int, N>;
template <bool B> using bool_c = std::integral_constant<bool, B>;

template <bool PRECISE, bool ROUND>
__device__ __forceinline__ void prefill_body(const PrefillParams& prm, const qm_kv_cache& cache,
                                             unsigned char* pf_smem, int qt, int pair) {
    PfStage* st = reinterpret_cast<PfStage*>(pf_smem);

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int col = lane & 31;       // MFMA column = (query row % 16, head)
    const int grp = lane >> 5;       // MFMA k / row group

    const int b = pair / prm.kv_heads;
    const int kvh = pair % prm.kv_heads;
    const int S = prm.seq;
    const int q_heads = 2 * prm.kv_heads;

    const int q0 = qt * kBM;
    const int my_row = q0 + 16 * wave + (col & 15);   // query row of this lane's column
    const int my_head = 2 * kvh + (col >> 4);
    const int wave_last_row = q0 + 16 * wave + 15;

    // ---- Q fragments (B operand): dims 16*kb + 8*grp .. +7 of this lane's column ----------------
    bf16x8_t qf[8];
    {
        const uint16_t* qp = prm.q + ((static_cast<int64_t>(b) * S + my_row) * q_heads + my_head) * kDim + 8 * grp;
#pragma unroll
        for (int kb = 0; kb < 8; ++kb) {
            uint4 raw = make_uint4(0, 0, 0, 0);
            if (my_row < S) raw = *reinterpret_cast<const uint4*>(qp + 16 * kb);
            qf[kb] = __builtin_bit_cast(bf16x8_t, raw);
        }
    }

    f32x16_t o[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[dt][r] = 0.0f;
    float m_run = -INFINITY;
    float l_run = 0.0f;

    const int64_t kv_base = static_cast<int64_t>(b) * prm.kv_stride_batch + static_cast<int64_t>(kvh) * prm.kv_stride_head;
    const int kv_row32 = static_cast<int>(prm.kv_stride_token);   // (the host rejects seq * stride >= 2^31)
    const int32_t* table = prm.page_table ? prm.page_table + static_cast<int64_t>(b) * prm.pages.max_pages : nullptr;

    // Global -> register staging of one K/V tile.  K: chunk c = tid + 256*i -> key c/16, dims
    // 8*(c%16).  V: thread (v_kg, v_dc) takes keys 4*v_kg..+3, dims 8*v_dc..+7.
    // (named registers, not arrays: an array here ends up as a stack object and every load is
    // followed by a wait and a scratch store)
    uint4 ks0, ks1, ks2, ks3, vs0, vs1, vs2, vs3;
    auto each_stage = [&](auto&& f) {
        f(ks0, vs0, 0);
        f(ks1, vs1, 1);
        f(ks2, vs2, 2);
        f(ks3, vs3, 3);
    };
    // The bits of tid are dealt so that 32 consecutive lanes hold 16 dim chunks x 2 key groups
    // whose transposed 8-byte LDS writes fall on 64 different banks: rows 16 apart have their
    // 8-slot blocks XOR-swizzled (which leaves the 16-lane fragment reads of 16 consecutive rows
    // conflict-free), rows 8 apart differ by 32 banks through the row stride, and the two key
    // groups differ by four slots.
    const int v_dc = tid & 15;
    const int v_kg = ((tid >> 5) & 1) | (((tid >> 4) & 1) << 1) | (((tid >> 6) & 3) << 2);
    const uint16_t* k_src = prm.k + kv_base + 8 * (tid & 15);
    const uint16_t* v_src = prm.v + kv_base + 8 * v_dc;
    const uint32_t k_lane_off = static_cast<uint32_t>((tid >> 4) * kv_row32);
    const uint32_t v_lane_off = static_cast<uint32_t>(4 * v_kg * kv_row32);
    auto load_tile = [&](int tile) {
        const int key0 = tile * kBN;
        if (key0 + kBN <= S) {
            const uint16_t* kt = k_src + static_cast<uint32_t>(key0 * kv_row32);
            const uint16_t* vt = v_src + static_cast<uint32_t>(key0 * kv_row32);
            each_stage([&](uint4& kk, uint4& vv, int i) {
                kk = *reinterpret_cast<const uint4*>(kt + (k_lane_off + static_cast<uint32_t>(16 * i * kv_row32)));
                vv = *reinterpret_cast<const uint4*>(vt + (v_lane_off + static_cast<uint32_t>(i * kv_row32)));
            });
        } else {
            // A key at or beyond S is redirected to the last key; such keys only occur in the
            // diagonal tile of the last query tile, where the causal mask removes them.
            each_stage([&](uint4& kk, uint4& vv, int i) {
                const int key = min(key0 + (tid >> 4) + 16 * i, S - 1);
                kk = *reinterpret_cast<const uint4*>(k_src + static_cast<uint32_t>(key * kv_row32));
                const int vkey = min(key0 + 4 * v_kg + i, S - 1);
                vv = *reinterpret_cast<const uint4*>(v_src + static_cast<uint32_t>(vkey * kv_row32));
            });
        }
    };
    // The block whose query tile equals the key tile also writes those K/V rows to the pages.
    // The eight page-table entries a thread needs for that are requested at the start of the
    // block (independent loads, long answered when the tile arrives); what is wrong with an
    // entry is kept as a status bit and reported once.
    int kp0 = -1, kp1 = -1, kp2 = -1, kp3 = -1, vp0 = -1, vp1 = -1, vp2 = -1, vp3 = -1;
    uint32_t page_err = 0;
    auto each_phys = [&](auto&& f) {
        f(kp0, vp0, 0);
        f(kp1, vp1, 1);
        f(kp2, vp2, 2);
        f(kp3, vp3, 3);
    };
    auto fetch_entry = [&](int key) -> int {
        if (key >= S) return -1;
        const int page = page_of(prm.pages, key);
        if (page >= prm.pages.max_pages) {
            page_err |= QM_STATUS_BAD_POSITION;
            return -1;
        }
        return table ? table[page] : page;
    };
    auto fetch_pages = [&]() {
        each_phys([&](int& kp, int& vp, int i) {
            kp = fetch_entry(qt * kBN + (tid >> 4) + 16 * i);
            vp = fetch_entry(qt * kBN + 4 * v_kg + i);
        });
    };
    auto page_store = [&](uint16_t* pool, int phys, int key, int dim0, const uint4& x) {
        if (key >= S || phys == -1) return;
        if (phys < 0 || phys >= cache.n_pages) {
            page_err |= QM_STATUS_BAD_PAGE;
            return;
        }
        const int page = page_of(prm.pages, key);
        const int64_t off = static_cast<int64_t>(phys) * cache.stride_page + static_cast<int64_t>(kvh) * cache.stride_head
                          + static_cast<int64_t>(key - page * prm.pages.page_size) * kDim;
        *reinterpret_cast<uint4*>(pool + off + dim0) = x;
    };
    auto write_pages = [&](int tile) {
        const int key0 = tile * kBN;
        uint4 k0, k1, k2, k3, v0, v1, v2, v3;
        each_stage([&](uint4& kk, uint4& vv, int i) {
            if (i == 0) { k0 = kk; v0 = vv; }
            if (i == 1) { k1 = kk; v1 = vv; }
            if (i == 2) { k2 = kk; v2 = vv; }
            if (i == 3) { k3 = kk; v3 = vv; }
        });
        each_phys([&](int& kp, int& vp, int i) {
            const uint4 kk = i == 0 ? k0 : i == 1 ? k1 : i == 2 ? k2 : k3;
            const uint4 vv = i == 0 ? v0 : i == 1 ? v1 : i == 2 ? v2 : v3;
            page_store(cache.k_pool, kp, key0 + (tid >> 4) + 16 * i, 8 * (tid & 15), kk);
            page_store(cache.v_pool, vp, key0 + 4 * v_kg + i, 8 * v_dc, vv);
        });
        if (page_err && prm.status) atomicOr(prm.status, page_err);
    };
    const int k_store = (tid >> 4) * kKS + 8 * (tid & 15);
    int v_store;
    {
        // transpose 4 keys x 8 dims -> 8 rows of 4 consecutive key slots; row d keeps its 8-slot
        // blocks XOR-swizzled by (d / 16) % 8.
        const int slot0 = 16 * (v_kg >> 2) + key_slot(4 * (v_kg & 3));
        const int phys = 8 * ((slot0 >> 3) ^ ((v_dc >> 1) & 7)) + (slot0 & 7);
        v_store = (8 * v_dc) * kVS + phys;
    }
    auto store_tile = [&](int stage) {
        uint16_t* kd = st[stage].k + k_store;
        each_stage([&](uint4& kk, uint4& vv, int i) {
            (void)vv;
            *reinterpret_cast<uint4*>(kd + 16 * i * kKS) = kk;
        });
        uint16_t* dst = st[stage].vt + v_store;
        auto put = [&](int e, uint32_t a, uint32_t b2, uint32_t c, uint32_t d) {
            const uint32_t sel = (e & 1) ? 0x07060302U : 0x05040100U;   // high or low halves of (second, first)
            uint2 packed;
            packed.x = __builtin_amdgcn_perm(b2, a, sel);
            packed.y = __builtin_amdgcn_perm(d, c, sel);
            *reinterpret_cast<uint2*>(dst + e * kVS) = packed;
        };
        put(0, vs0.x, vs1.x, vs2.x, vs3.x);
        put(1, vs0.x, vs1.x, vs2.x, vs3.x);
        put(2, vs0.y, vs1.y, vs2.y, vs3.y);
        put(3, vs0.y, vs1.y, vs2.y, vs3.y);
        put(4, vs0.z, vs1.z, vs2.z, vs3.z);
        put(5, vs0.z, vs1.z, vs2.z, vs3.z);
        put(6, vs0.w, vs1.w, vs2.w, vs3.w);
        put(7, vs0.w, vs1.w, vs2.w, vs3.w);
    };

    // ---- the pieces of one 32-key chunk --------------------------------------------------------------
    // S^T = K Q^T of chunk `half` of a stage: rows = 32 keys, cols = 32 (row, head) columns.
    const int k_lane = col * kKS + 8 * grp;
    auto qk = [&](int stage, auto half, f32x16_t& s) {
        const uint16_t* kp = st[stage].k + k_lane + 32 * decltype(half)::value * kKS;
        bf16x8_t kf[8];
#pragma unroll
        for (int kb = 0; kb < 8; ++kb) kf[kb] = lds_frag(kp + 16 * kb);
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = 0.0f;
#pragma unroll
        for (int kb = 0; kb < 8; ++kb) s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[kb], qf[kb], s, 0, 0, 0);
    };
    // V^T fragment of (chunk half h, group kg, dim tile dt), lane (col, grp): row d = 32*dt + col,
    // slot block (4h + 2kg + grp) ^ ((d / 16) % 8); the lane part and the constant part of that XOR
    // touch different bits.
    const int v_lane = col * kVS + 8 * (grp ^ (col >> 4));
    auto v_frags = [&](int stage, auto half, bf16x8_t (&vf)[8]) {
        constexpr int h = decltype(half)::value;
        const uint16_t* vp = st[stage].vt + v_lane;
#pragma unroll
        for (int j = 0; j < 8; ++j)
            vf[j] = lds_frag(vp + 32 * (j & 3) * kVS + 8 * ((4 * h + 2 * (j >> 2)) ^ (2 * (j & 3))));
    };
    // O^T += V^T P^T for one chunk: two 16-key groups x four 32-dim tiles.  On the diagonal a
    // 16-key group that lies wholly after the wave's last row is masked for every column: it is
    // skipped, so that later tokens are not even multiplied by zero.
    auto pv = [&](const bf16x8_t (&vf)[8], const PFrag& p, auto diag, int key_base) {
#pragma unroll
        for (int kg = 0; kg < 2; ++kg) {
            if (decltype(diag)::value && key_base + 16 * kg > wave_last_row) continue;
#pragma unroll
            for (int dt = 0; dt < 4; ++dt) {
                o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[4 * kg + dt], p.hi[kg], o[dt], 0, 0, 0);
                if (PRECISE) o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[4 * kg + dt], p.lo[kg], o[dt], 0, 0, 0);
            }
        }
    };
    // Softmax works in `units`: rounded scaled scores (ROUND) or raw fp32 dot products, whose
    // scale is folded into the exponent's multiplier (the host admits only scale > 0 there).
    const float coef = ROUND ? kLog2e : prm.scale * kLog2e;
    const float slack = ROUND ? kRescaleSlack : kRescaleSlack / prm.scale;
    // Score roundings and causal mask in place; returns the column maximum.
    auto scores = [&](f32x16_t& s, auto masked, int key_base) -> float {
        // accumulator register r of lane group grp is key key_base + 8*(r/4) + 4*grp + r%4
        const int lim = my_row - key_base - 4 * grp;
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
            float x0 = s[r], x1 = s[r + 1];
            if (ROUND) {
                round_bf16_pair(x0, x1, x0, x1);
                round_bf16_pair(x0 * prm.scale, x1 * prm.scale, x0, x1);
            }
            if (decltype(masked)::value) {
                const int e = 8 * (r >> 2) + (r & 3);
                if (e > lim) x0 = -INFINITY;
                if (e + 1 > lim) x1 = -INFINITY;
            }
            s[r] = x0;
            s[r + 1] = x1;
            mx = fmaxf(mx, fmaxf(x0, x1));
        }
        return halves_max(mx);
    };
    // Raise the running maximum if some column of the wave exceeds it by more than the slack,
    // and rescale O and the running sum for it.
    float m_scaled = 0.0f;
    auto update_max = [&](float mx) {
        const bool need = __builtin_amdgcn_ballot_w64(mx > m_run + slack) != 0;
        if (need) {
            const float m_new = fmaxf(m_run, mx);
            const float m_ref = m_new == -INFINITY ? 0.0f : m_new;
            const float alpha = fast_exp2((m_run - m_ref) * coef);
            m_run = m_new;
            m_scaled = m_ref * coef;
            l_run *= alpha;
#pragma unroll
            for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) o[dt][r] *= alpha;
        }
    };
    // P = exp(score - max) as bf16 B operands; adds this lane's share of the row sum.
    auto probs = [&](const f32x16_t& s, PFrag& p) {
        uint32_t hi[8], lo[8];
        float psum = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
            const float e0 = fast_exp2(fmaf(s[r], coef, -m_scaled));
            const float e1 = fast_exp2(fmaf(s[r + 1], coef, -m_scaled));
            hi[r >> 1] = pack_bf16_pair(e0, e1);
            if (PRECISE) {
                lo[r >> 1] = pack_bf16_pair(e0 - lo_bf16(hi[r >> 1]), e1 - hi_bf16(hi[r >> 1]));
                psum += e0 + e1;
            } else {
                psum = dot2_bf16(hi[r >> 1], 0x3f803f80U, psum);   // the sum of what the MFMA multiplies
            }
        }
#pragma unroll
        for (int kg = 0; kg < 2; ++kg) {
            p.hi[kg] = __builtin_bit_cast(bf16x8_t, make_uint4(hi[4 * kg], hi[4 * kg + 1], hi[4 * kg + 2], hi[4 * kg + 3]));
            if (PRECISE)
                p.lo[kg] = __builtin_bit_cast(bf16x8_t, make_uint4(lo[4 * kg], lo[4 * kg + 1], lo[4 * kg + 2], lo[4 * kg + 3]));
        }
        l_run += psum;
    };
    auto chunk = [&](int stage, auto half, auto diag, int key_base) {
        // On the diagonal a wave whose last row precedes this chunk has nothing to do in it.
        if (decltype(diag)::value && key_base > wave_last_row) return;
        f32x16_t s;
        bf16x8_t vf[8];
        PFrag p;
        qk(stage, half, s);
        v_frags(stage, half, vf);   // requested before the softmax arithmetic, used after it
        const float mx = scores(s, diag, key_base);
        update_max(mx);
        probs(s, p);
        pv(vf, p, diag, key_base);
    };

    // ---- tile 0 into stage 0, then the key tiles up to the diagonal ---------------------------------
    load_tile(0);
    if (prm.has_cache) fetch_pages();
    if (prm.has_cache && qt == 0) write_pages(0);
    store_tile(0);
    __syncthreads();

    if (!PRECISE) {
        for (int t = 0; t < qt; ++t) {
            const int stage = t & 1;
            load_tile(t + 1);
            chunk(stage, int_c<0>{}, bool_c<false>{}, 0);
            chunk(stage, int_c<1>{}, bool_c<false>{}, 0);
            if (prm.has_cache && t + 1 == qt) write_pages(qt);
            store_tile(stage ^ 1);
            __syncthreads();
        }
    }
    chunk(qt & 1, int_c<0>{}, bool_c<true>{}, qt * kBN);
    chunk(qt & 1, int_c<1>{}, bool_c<true>{}, qt * kBN + 32);
    __syncthreads();   // the stages become the output staging area

    // ---- normalise, stage through LDS, write 16 bytes per lane -------------------------------------
    const float l_tot = halves_sum(l_run);
    const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
    uint16_t* stage = reinterpret_cast<uint16_t*>(pf_smem) + wave * 32 * kOS;   // 32 columns x 128 dims per wave
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
            const int d0 = 32 * dt + 8 * rq + 4 * grp;
            uint2 packed;
            packed.x = pack_bf16_pair(o[dt][4 * rq + 0] * inv, o[dt][4 * rq + 1] * inv);
            packed.y = pack_bf16_pair(o[dt][4 * rq + 2] * inv, o[dt][4 * rq + 3] * inv);
            *reinterpret_cast<uint2*>(&stage[col * kOS + d0]) = packed;
        }
    }
    __builtin_amdgcn_s_waitcnt(0);   // the wave reads back only what it wrote itself
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int it = 0; it < 8; ++it) {
        const int c = 4 * it + (lane >> 4);
        const int chunk = lane & 15;
        const int row = q0 + 16 * wave + (c & 15);
        const int head = 2 * kvh + (c >> 4);
        if (row < S) {
            const uint4 val = *reinterpret_cast<const uint4*>(&stage[c * kOS + 8 * chunk]);
            *reinterpret_cast<uint4*>(prm.out + ((static_cast<int64_t>(b) * S + row) * q_heads + head) * kDim + 8 * chunk) = val;
        }
    }
}

// grid = batch * kv_heads * n_qtiles blocks, heaviest query tile first.  The first query tile
// takes the split-precision P path.
template <bool ROUND>
__global__ __launch_bounds__(kPfThreads, 2) void prefill_causal_kernel(PrefillParams prm, qm_kv_cache cache) {
    extern __shared__ __attribute__((aligned(16))) unsigned char pf_smem[];
    const int pairs = prm.batch * prm.kv_heads;
    const int bid = blockIdx.x;
    const int qt = prm.n_qtiles - 1 - bid / pairs;
    const int pair = bid % pairs;
    if (qt == 0) {
        prefill_body<true, ROUND>(prm, cache, pf_smem, 0, pair);
    } else {
        prefill_body<false, ROUND>(prm, cache, pf_smem, qt, pair);
    }
}

}  // namespace qm

extern "C" int32_t qm_prefill_attention_causal(
    const uint16_t* query, const uint16_t* key, const uint16_t* value,
    uint16_t* context_out,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    int32_t batch, int32_t seq, int32_t q_heads, int32_t kv_heads, float scale,
    int64_t kv_stride_token, int64_t kv_stride_head, int64_t kv_stride_batch,
    uint32_t* status_dev, void* hip_stream) {
    using namespace qm;
    if (kv_stride_token == 0 && kv_stride_head == 0 && kv_stride_batch == 0) {
        kv_stride_token = static_cast<int64_t>(kv_heads) * kDim;     // [batch][seq][kv_heads][128]
        kv_stride_head = kDim;
        kv_stride_batch = static_cast<int64_t>(seq) * kv_heads * kDim;
    }
    if (kv_stride_token < kDim || kv_stride_head < 0 || kv_stride_batch < 0
        || ((kv_stride_token | kv_stride_head | kv_stride_batch) & 7))
        return QM_ERR_GEOMETRY;
    if (static_cast<int64_t>(seq) * kv_stride_token >= (1LL << 31)) return QM_ERR_ARGUMENT;
    if (!query || !key || !value || !context_out) return QM_ERR_NULL;
    if (batch < 0 || seq < 0) return QM_ERR_ARGUMENT;
    if (kv_heads <= 0 || q_heads != 2 * kv_heads) return QM_ERR_GEOMETRY;   // GQA pair on the MFMA columns
    const uintptr_t align = reinterpret_cast<uintptr_t>(query) | reinterpret_cast<uintptr_t>(key)
                          | reinterpret_cast<uintptr_t>(value) | reinterpret_cast<uintptr_t>(context_out);
    if (align & 15) return QM_ERR_GEOMETRY;
    qm_kv_cache desc = {};
    PageMap pm = make_page_map(16, 1);
    if (cache) {
        const int32_t rc = check_cache(cache, max_pages);
        if (rc != QM_OK) return rc;
        if (cache->kv_heads != kv_heads) return QM_ERR_GEOMETRY;
        if (seq > cache_capacity(cache, max_pages)) return QM_ERR_SLOT_RANGE;
        if (!page_table && (batch > 1 || (seq > 0 && (seq - 1) / cache->page_size >= cache->n_pages)))
            return QM_ERR_SLOT_RANGE;   // an identity table can serve one sequence only
        desc = *cache;
        pm = make_page_map(cache->page_size, max_pages);
    }
    if (batch == 0 || seq == 0) return QM_OK;
    const int n_qtiles = (seq + kBM - 1) / kBM;
    const int64_t pairs = static_cast<int64_t>(batch) * kv_heads;
    if (pairs * n_qtiles > 0x7fffffffLL) return QM_ERR_ARGUMENT;

    PrefillParams prm;
    prm.q = query; prm.k = key; prm.v = value; prm.out = context_out;
    prm.page_table = page_table; prm.status = status_dev; prm.pages = pm;
    prm.has_cache = cache ? 1 : 0;
    prm.kv_stride_token = kv_stride_token; prm.kv_stride_head = kv_stride_head; prm.kv_stride_batch = kv_stride_batch;
    prm.batch = batch; prm.seq = seq; prm.kv_heads = kv_heads; prm.n_qtiles = n_qtiles; prm.scale = scale;

    hipStream_t s = static_cast<hipStream_t>(hip_stream);
    const size_t smem = sizeof(PfStage) * kPfStages;
    const bool round_scores = option_value(QM_OPT_PREFILL_SCORE_ROUNDING) != 0;
    if (!round_scores && !(scale > 0.0f)) return QM_ERR_ARGUMENT;   // the scale is folded into the exponent there
    const auto kernel = round_scores ? prefill_causal_kernel<true> : prefill_causal_kernel<false>;
    static std::atomic<bool> lds_raised[2][kMaxDevices];
    const int32_t rc_lds = ensure_dynamic_lds(reinterpret_cast<const void*>(kernel), static_cast<int>(smem),
                                              lds_raised[round_scores ? 1 : 0]);
    if (rc_lds != QM_OK) return rc_lds;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(pairs * n_qtiles)), dim3(kPfThreads), smem, s, prm, desc);
    return launch_status();
}
