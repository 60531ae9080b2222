// qm_prefill.hip — causal GQA prefill attention on gfx950 bf16 MFMA, fused with the paged K/V write.
//
// Tiling.  A block of four waves owns 64 query rows of one (batch, kv head) and both query heads
// of the GQA pair: a wave's MFMA column dimension is 32 = 16 rows x 2 heads, so every K and V
// fragment read from LDS feeds both heads.  Keys are streamed in tiles of 64 through two LDS
// buffers (global loads for the next tile are in flight while the current one is multiplied).
// A wave computes S^T = K Q^T with v_mfma_f32_32x32x16_bf16 (keys on MFMA rows, query columns on
// lanes), so that the softmax statistics of a query column live in one lane pair, and the
// accumulator layout of S^T is directly the B-operand layout of O^T += V^T P^T.  V is transposed
// on its way into LDS ([dim][key slot], key slots permuted to match the accumulator layout).
// (QM_PF_KSPLIT=2 builds blocks of two wave groups that take alternate key tiles and merge their
// softmax states through LDS at the end: it shortens the longest block by 15 % but two waves of
// one block then share each SIMD, and the batch-4 x 1024 case measured 8 % slower.)
//
// Scheduling.  Blocks are numbered heaviest query tile first; the hardware hands the next
// (lighter) block to whichever CU retires one.  Blocks that share K/V differ by a multiple of
// batch*kv_heads and therefore land on the same XCD and hit its L2.
//
// Rounding.  Scores are rounded to bf16 before and after scaling like the reference
// (R17:15879-15890); softmax runs online in fp32; P enters the P.V MFMA as bf16 — except in the
// first query tile, whose rows have so few keys that outputs are large: there P is split into
// hi + lo bf16 parts (two MFMAs) to stay inside the 1e-2 output tolerance.
//
// Causality.  A key after a query row never contributes; keys of later 16-row groups are not
// read into the product at all.  Inside a wave's own 16-row diagonal group the mask is P = 0
// times V, so a non-finite V of a later row of the same group would propagate (the reference
// skips those keys; finite values, the only ones a prefill produces, behave identically).
//
// Algorithmic work per (batch, kv head): flops = 2 heads * 2 matmuls * 2 * 128 * S(S+1)/2;
// HBM bytes = Q + O (2 heads) + K + V read once + K + V written to pages.  Bound: MFMA (with the
// softmax VALU work — 16 exponentials per lane per 32 keys — as the practical limiter).

#include "qm_device.h"
#include "qm_host.h"

#include <type_traits>

// Build-time variants kept for measurement: how many wave groups split the key tiles of a block
// (1 or 2); how many LDS fragment reads are requested ahead of the MFMAs (0 none, 1 K, 2 K and
// V^T); waves per SIMD.
#ifndef QM_PF_KSPLIT
#define QM_PF_KSPLIT 1
#endif
#ifndef QM_PF_PREFETCH
#define QM_PF_PREFETCH 2
#endif
#ifndef QM_PF_MINWAVES
#define QM_PF_MINWAVES 2
#endif

namespace qm {

constexpr int kPfGroup = 256;                    // threads of one wave group
constexpr int kPfThreads = kPfGroup * QM_PF_KSPLIT;
constexpr int kBM = 64;          // query rows per block
constexpr int kBN = 64;          // keys per tile
constexpr int kKS = kDim + 8;    // LDS row stride of the K tile (elements)
constexpr int kVS = kBN + 8;     // LDS row stride of the V^T tile (elements)
constexpr int kOS = kDim + 8;    // LDS row stride of the output staging tile

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

struct PfShared {
    uint16_t k[2][kBN * kKS];
    uint16_t vt[2][kDim * kVS];
};

// LDS slot of key j (0..15) inside a 16-key group: MFMA k index 8*g + e holds the key that the
// S^T accumulator register e of lane group g belongs to.
__device__ __forceinline__ int key_slot(int j) {
    return 8 * ((j & 7) >> 2) + 4 * (j >> 3) + (j & 3);
}

__device__ __forceinline__ bf16x8_t lds_frag(const uint16_t* p) {
    return *reinterpret_cast<const bf16x8_t*>(p);
}

template <bool PRECISE>
__device__ __forceinline__ void prefill_body(const PrefillParams& prm, const qm_kv_cache& cache,
                                             unsigned char* pf_smem, int qt, int pair) {
    // Wave group kp (0 .. KSPLIT-1) owns key tiles kp, kp + KSPLIT, ...; it has its own pair of
    // LDS tile buffers and its own online-softmax state, merged through LDS at the end.
    const int kp = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) >> 8);
    PfShared& sh = reinterpret_cast<PfShared*>(pf_smem)[kp];

    const int tid = threadIdx.x & (kPfGroup - 1);
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
    const int64_t kv_row = prm.kv_stride_token;
    const int kv_row32 = static_cast<int>(kv_row);
    const int32_t* table = prm.page_table ? prm.page_table + static_cast<int64_t>(b) * prm.pages.max_pages : nullptr;

    // Global -> register staging of one K/V tile.  K: chunk c = tid + 256*i -> key c/16, dims
    // 8*(c%16).  V: thread (kg = tid/16, dc = tid%16) takes keys 4*kg..4*kg+3, dims 8*dc..+7.
    // (named registers, not arrays: an array here ends up as a stack object and every load is
    // followed by a wait and a scratch store)
    uint4 ks0, ks1, ks2, ks3, vs0, vs1, vs2, vs3;
    auto each_stage = [&](auto&& f) {
        f(ks0, vs0, 0);
        f(ks1, vs1, 1);
        f(ks2, vs2, 2);
        f(ks3, vs3, 3);
    };
    // V staging: thread (v_kg, v_dc) takes keys 4*v_kg..+3, dims 8*v_dc..+7.  The bits of tid are dealt
    // so that 32 consecutive lanes hold 16 dim chunks x 2 key groups whose transposed 8-byte LDS
    // writes fall on 64 different banks: rows 16 apart have their 8-slot blocks XOR-swizzled (which
    // leaves the 16-lane fragment reads of 16 consecutive rows conflict-free), rows 8 apart differ by
    // 32 banks through the row stride, and the two key groups differ by four slots.
    const int v_dc = tid & 15;
    const int v_kg = ((tid >> 5) & 1) | (((tid >> 4) & 1) << 1) | (((tid >> 6) & 3) << 2);
    const uint16_t* k_src = prm.k + kv_base + 8 * (tid & 15);
    const uint16_t* v_src = prm.v + kv_base + 8 * v_dc;
    // Unpredicated: a key at or beyond S is redirected to the last key; such keys only occur in the
    // diagonal tile of the last query tile, where the causal mask removes them (key > row).
    auto load_tile = [&](int tile) {
        const int key0 = tile * kBN;
        each_stage([&](uint4& kk, uint4& vv, int i) {
            // (32-bit element offsets: the host rejects seq * stride >= 2^31)
            const int key = min(key0 + (tid >> 4) + 16 * i, S - 1);
            kk = *reinterpret_cast<const uint4*>(k_src + static_cast<uint32_t>(key * kv_row32));
            const int vkey = min(key0 + 4 * v_kg + i, S - 1);
            vv = *reinterpret_cast<const uint4*>(v_src + static_cast<uint32_t>(vkey * kv_row32));
        });
    };
    // The block whose query tile equals the key tile also writes those K/V rows to the pages.
    auto write_pages = [&](int tile) {
        const int key0 = tile * kBN;
        each_stage([&](uint4& kk, uint4& vv, int i) {
            const int key = key0 + (tid >> 4) + 16 * i;
            if (key < S) {
                const int64_t off = tile_offset(cache, prm.pages, table, key, kvh, prm.status);
                if (off >= 0) *reinterpret_cast<uint4*>(cache.k_pool + off + 8 * (tid & 15)) = kk;
            }
            const int vkey = key0 + 4 * v_kg + i;
            if (vkey < S) {
                const int64_t off = tile_offset(cache, prm.pages, table, vkey, kvh, prm.status);
                if (off >= 0) *reinterpret_cast<uint4*>(cache.v_pool + off + 8 * v_dc) = vv;
            }
        });
    };
    auto store_tile = [&](int buf) {
        each_stage([&](uint4& kk, uint4& vv, int i) {
            (void)vv;
            *reinterpret_cast<uint4*>(&sh.k[buf][((tid >> 4) + 16 * i) * kKS + 8 * (tid & 15)]) = kk;
        });
        // transpose 4 keys x 8 dims -> 8 rows of 4 consecutive key slots; row d keeps its 8-slot
        // blocks XOR-swizzled by (d / 16) % 8.
        const int slot0 = 16 * (v_kg >> 2) + key_slot(4 * (v_kg & 3));
        const int phys = 8 * ((slot0 >> 3) ^ ((v_dc >> 1) & 7)) + (slot0 & 7);
        uint16_t* dst = &sh.vt[buf][(8 * v_dc) * kVS + phys];
        auto put = [&](int e, uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
            uint2 packed;
            if (e & 1) {
                packed.x = (a >> 16) | (b & 0xffff0000U);
                packed.y = (c >> 16) | (d & 0xffff0000U);
            } else {
                packed.x = (a & 0xffffU) | (b << 16);
                packed.y = (c & 0xffffU) | (d << 16);
            }
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

    // Both groups run the same number of iterations (the barrier is block-wide); a group whose
    // tile index runs past the diagonal idles through the last one.
    const int n_iter = qt / QM_PF_KSPLIT + 1;
    if (kp <= qt) {
        load_tile(kp);
        if (prm.has_cache && kp == qt) write_pages(kp);
        store_tile(0);
    }
    __syncthreads();

    for (int it = 0; it < n_iter; ++it) {
        const int tile = it * QM_PF_KSPLIT + kp;
        const int buf = it & 1;
        const bool more = tile + QM_PF_KSPLIT <= qt;
        if (more) {
            load_tile(tile + QM_PF_KSPLIT);
            if (prm.has_cache && tile + QM_PF_KSPLIT == qt) write_pages(tile + QM_PF_KSPLIT);
        }
        if (tile <= qt) {
        const bool diagonal = tile == qt;

#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int key_base = tile * kBN + 32 * half;
            // On the diagonal a wave whose last row precedes this half has nothing to do there.
            if (diagonal && key_base > q0 + 16 * wave + 15) continue;

            // ---- S^T = K Q^T : rows = 32 keys, cols = 32 (row, head) columns ----------------------
            f32x16_t s;
#pragma unroll
            for (int r = 0; r < 16; ++r) s[r] = 0.0f;
            const uint16_t* kp = &sh.k[buf][(32 * half + col) * kKS + 8 * grp];
            // All eight K fragments are requested before the first MFMA, and the eight V^T
            // fragments of this half before the softmax arithmetic, so that LDS latency is paid
            // once per phase instead of once per MFMA.
#if QM_PF_PREFETCH >= 1
            bf16x8_t kfr[8];
#pragma unroll
            for (int kb = 0; kb < 8; ++kb) kfr[kb] = lds_frag(kp + 16 * kb);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int kb = 0; kb < 8; ++kb) {
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfr[kb], qf[kb], s, 0, 0, 0);
            }
#else
#pragma unroll
            for (int kb = 0; kb < 8; ++kb) {
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lds_frag(kp + 16 * kb), qf[kb], s, 0, 0, 0);
            }
#endif
            bf16x8_t vfr[2][4];
#if QM_PF_PREFETCH >= 2
#pragma unroll
            for (int kg = 0; kg < 2; ++kg) {
                const int sb = 4 * half + 2 * kg + grp;
#pragma unroll
                for (int dt = 0; dt < 4; ++dt) {
                    const int d = 32 * dt + col;
                    vfr[kg][dt] = lds_frag(&sh.vt[buf][d * kVS + 8 * (sb ^ ((d >> 4) & 7))]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#endif

            // ---- reference score roundings, causal mask, online softmax ---------------------------
            float mx = -INFINITY;
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
                float x0, x1;
                round_bf16_pair(s[r], s[r + 1], x0, x1);
                round_bf16_pair(x0 * prm.scale, x1 * prm.scale, x0, x1);
                if (diagonal) {
                    const int key = key_base + 8 * (r >> 2) + 4 * grp + (r & 3);
                    if (key > my_row) x0 = -INFINITY;
                    if (key + 1 > my_row) x1 = -INFINITY;
                }
                s[r] = x0;
                s[r + 1] = x1;
                mx = fmaxf(mx, fmaxf(x0, x1));
            }
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float m_new = fmaxf(m_run, mx);
            const float m_ref = m_new == -INFINITY ? 0.0f : m_new;
            if (__builtin_amdgcn_ballot_w64(m_new > m_run)) {
                const float alpha = fast_exp2((m_run - m_ref) * kLog2e);
                l_run *= alpha;
#pragma unroll
                for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) o[dt][r] *= alpha;
            }
            m_run = m_new;
            const float m_scaled = m_ref * kLog2e;
            float psum = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                s[r] = fast_exp2(fmaf(s[r], kLog2e, -m_scaled));
                psum += s[r];
            }
            l_run += psum;

            // ---- O^T += V^T P^T : two 16-key groups x four 32-dim tiles ---------------------------
#pragma unroll
            for (int kg = 0; kg < 2; ++kg) {
                // A 16-key group that lies wholly after the wave's last row is masked for every
                // column: skip it, so that later tokens are not even multiplied by zero.
                if (diagonal && key_base + 16 * kg > q0 + 16 * wave + 15) continue;
                bf16x8_t phi, plo;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float pv = s[8 * kg + e];
                    phi[e] = static_cast<__bf16>(pv);
                    if (PRECISE) plo[e] = static_cast<__bf16>(pv - static_cast<float>(phi[e]));
                }
#if QM_PF_PREFETCH < 2
                {
                    const int sb = 4 * half + 2 * kg + grp;
#pragma unroll
                    for (int dt = 0; dt < 4; ++dt) {
                        const int d = 32 * dt + col;
                        vfr[kg][dt] = lds_frag(&sh.vt[buf][d * kVS + 8 * (sb ^ ((d >> 4) & 7))]);
                    }
                }
#endif
#pragma unroll
                for (int dt = 0; dt < 4; ++dt) {
                    o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vfr[kg][dt], phi, o[dt], 0, 0, 0);
                    if (PRECISE) o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vfr[kg][dt], plo, o[dt], 0, 0, 0);
                }
            }
        }

        }   // tile <= qt

        if (more) store_tile(buf ^ 1);
        __syncthreads();
    }

#if QM_PF_KSPLIT == 2
    // ---- merge the two key groups: group 1 hands its (O, max, sum) to group 0 through LDS --------
    {
        float* xo = reinterpret_cast<float*>(pf_smem);                 // [wave][64 regs][64 lanes]
        float* xm = xo + 4 * 64 * 64;                                  // [wave][2][64 lanes]
        if (kp == 1) {
#pragma unroll
            for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) xo[(wave * 64 + dt * 16 + r) * 64 + lane] = o[dt][r];
            xm[(wave * 2 + 0) * 64 + lane] = m_run;
            xm[(wave * 2 + 1) * 64 + lane] = l_run;
        }
        __syncthreads();
        if (kp == 1) return;
        const float m1 = xm[(wave * 2 + 0) * 64 + lane];
        const float l1 = xm[(wave * 2 + 1) * 64 + lane];
        const float mm = fmaxf(m_run, m1);
        const float m_ref = mm == -INFINITY ? 0.0f : mm;
        const float a0 = fast_exp2((m_run - m_ref) * kLog2e);
        const float a1 = fast_exp2((m1 - m_ref) * kLog2e);
        l_run = l_run * a0 + l1 * a1;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                o[dt][r] = fmaf(o[dt][r], a0, xo[(wave * 64 + dt * 16 + r) * 64 + lane] * a1);
    }
    constexpr int kStageOffset = 4 * 64 * 64 * 4 + 4 * 2 * 64 * 4;   // bytes, behind the exchange area
#else
    constexpr int kStageOffset = 0;
#endif

    // ---- normalise, stage through LDS, write 16 bytes per lane -------------------------------------
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
    uint16_t* stage = reinterpret_cast<uint16_t*>(pf_smem + kStageOffset) + wave * 32 * kOS;   // 32 columns x 128 dims per wave
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
            const int d0 = 32 * dt + 8 * rq + 4 * grp;
            uint2 packed;
            packed.x = static_cast<uint32_t>(f2bf(o[dt][4 * rq + 0] * inv))
                     | (static_cast<uint32_t>(f2bf(o[dt][4 * rq + 1] * inv)) << 16);
            packed.y = static_cast<uint32_t>(f2bf(o[dt][4 * rq + 2] * inv))
                     | (static_cast<uint32_t>(f2bf(o[dt][4 * rq + 3] * inv)) << 16);
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

// grid = batch * kv_heads * n_qtiles blocks, heaviest query tile first: the hardware hands the
// next (lighter) block to whichever CU retires one, which pairs heavy with light tiles.  The
// first query tile takes the split-precision P path.
__global__ __launch_bounds__(kPfThreads, QM_PF_MINWAVES) void prefill_causal_kernel(PrefillParams prm, qm_kv_cache cache) {
    extern __shared__ __attribute__((aligned(16))) unsigned char pf_smem[];
    const int pairs = prm.batch * prm.kv_heads;
    const int bid = blockIdx.x;
    const int qt = prm.n_qtiles - 1 - bid / pairs;
    const int pair = bid % pairs;
    if (qt == 0) {
        prefill_body<true>(prm, cache, pf_smem, 0, pair);
    } else {
        prefill_body<false>(prm, cache, pf_smem, qt, pair);
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
    const size_t smem = sizeof(PfShared) * QM_PF_KSPLIT;
    static bool attr_set = false;
    if (!attr_set) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(prefill_causal_kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem));
        if (e != hipSuccess) return hip_code(e);
        attr_set = true;
    }
    hipLaunchKernelGGL(prefill_causal_kernel, dim3(static_cast<unsigned>(pairs * n_qtiles)), dim3(kPfThreads), smem, s,
                       prm, desc);
    return launch_status();
}
