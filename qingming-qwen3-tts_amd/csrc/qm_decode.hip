// qm_decode.hip — GQA decode attention (single stream and ragged multi-stream) for gfx950.
//
// Work decomposition.  The context of one (stream, kv head) is cut into tiles of 16 tokens
// (= one native page, 4 KiB of K and 4 KiB of V, contiguous).  A block of four waves owns
// `tiles_per_block` consecutive tiles (split-K); its waves take tiles round-robin.  Inside a
// wave a tile is fetched by four 128-bit loads per lane for K and four for V: load i covers
// tokens 4i..4i+3, lane l reads token 4i + l/16, dimensions 8*(l%16)..+7 — one instruction
// reads 1 KiB contiguous.  All query heads that share the kv head (GQA group G) are served
// from the same registers, so K and V are read from HBM exactly once.
//
// Each 16-lane DPP row is an independent online-softmax stream: its score is completed by a
// row-rotate all-reduce, and it keeps its own running (max, sum, acc[G][8 dims per lane]).
// The 16 row-streams of a block are merged through LDS; blocks write fp32 partials
// (acc, max, sum) to the caller's workspace and a small second kernel merges the splits.
// Blocks are dispatched by the hardware as earlier ones retire, which balances ragged lengths;
// letting the last block to arrive at a per-(stream, head) counter merge in place needs one
// device-scope fence per block (write-back and invalidate of the XCD's L2): measured, with
// bit-identical results, at 17 us instead of 6.6 us for one stream of 512 tokens and 17x slower
// on the ragged batch (a persistent variant pulling work items from a counter: 8x slower), so the
// merge stays a second launch.
//
// Rounding: scores are rounded to bf16 before and after scaling as the reference does
// (R17:16102-16116); probabilities stay fp32 (the reference's bf16(P) after a full-row
// softmax, R17:16136-16141, cannot be formed by a single-pass kernel).
//
// Algorithmic HBM bytes per token of context: kv_heads * 128 * 2 B * 2 (K and V) = 4096 B
// at 8 kv heads; the kernel is bound by HBM bandwidth.

#include "qm_device.h"
#include "qm_host.h"
#include "qm_norm_rope_head.h"
#include "qm_decode_step.h"

#include <stdlib.h>

#include <atomic>

namespace qm {

constexpr int kDecodeThreads = 256;
constexpr int kDecodeWaves = 4;
constexpr int kRowStreams = 16;  // 4 waves x 4 DPP rows
constexpr int kMaxTilesPerBlock = 64;
constexpr int kMergeRound = kDecodeMergeRound;   // splits merged per round of loads in the merge kernel
// Calls whose contexts may exceed this many bytes (streams x max_seq_len x bytes per token) read
// K and V with the non-temporal hint.  Ragged batches of 256..4096 tokens, plain / non-temporal:
// 16 streams (156 MiB read, bound 256 MiB) 32.5 / 32.8 us, 32 (290, 512) 54.2 / 55.2 us,
// 48 (429, 768) 89.8 / 78.2 us, 64 (588, 1024) 119.4 / 104.9 us, 128 (1074, 2048) 210.5 / 190.5 us:
// below about twice the 256 MiB last-level cache part of a context is still cached from the
// step before and plain loads find it there.
constexpr int64_t kStreamingContextBytes = 512ll << 20;

struct DecodeParams {
    const uint16_t* query;        // [n_streams][q_heads][128]
    uint16_t* out;                // [n_streams][q_heads][128]
    const int32_t* page_table;    // [n_streams][max_pages] or NULL
    const int32_t* seq_lens;      // [n_streams] or NULL (single stream: fixed range)
    float* partial;               // workspace
    uint32_t* status;
    PageMap pages;
    int max_seq_len;
    int fixed_key_start;
    int fixed_key_end;
    int tiles_per_block;
    int max_splits;
    int q_heads;
    float scale;
    // Fused decode step (single stream): the raw projections of the new token; the kernel norms and
    // rotates q itself and appends k, v at `step_position` before attending.
    const uint16_t* step_q;       // [q_heads][128]
    const uint16_t* step_k;       // [kv_heads][128]
    const uint16_t* step_v;       // [kv_heads][128]
    const uint16_t* step_q_norm;  // [128]
    const uint16_t* step_k_norm;  // [128]
    const uint16_t* step_cos;     // [128]
    const uint16_t* step_sin;     // [128]
    uint16_t* step_q_rotated;     // [q_heads][128] or NULL
    int step_position;
    float step_epsilon;
    // Blocks (in y) that share one kv head: 1 when the kernel's G is the whole GQA group; a group the kernels
    // are not instantiated for runs as several blocks of G heads each on the same K and V.
    int head_groups_per_kv;
    // Rows of one sequence as streams (qm_attention_rows): stream i is query row i, all rows share one page
    // table, row i attends keys [window start, rows_cache_before + i + 1).  -1 = off.
    int rows_cache_before;
    int rows_window;
};

// Partial record of one (stream, kv head, split): G*128 acc, G max, G sum.
template <int G>
__host__ __device__ constexpr int partial_floats() { return G * kDim + 2 * G; }

// Key range [start, end) of row `stream` of one sequence (GENERIC kernels, rows_cache_before >= 0): R17:15784-15789.
__device__ __forceinline__ void row_key_range(const DecodeParams& prm, int stream, int& key_start, int& key_end) {
    key_end = prm.rows_cache_before + stream + 1;
    key_start = prm.rows_window > 0 ? max(key_end - prm.rows_window, 0) : 0;
}

// 16 bytes of K or V.  STREAMING adds the non-temporal hint: contexts much larger than the caches
// are read once per step and should not displace anything on their way (measured on a 600 MB
// read: 6.7-7.0 TB/s against 6.0-6.5 TB/s with plain loads).
template <bool STREAMING>
__device__ __forceinline__ uint4 kv_load(const uint16_t* p) {
    if (STREAMING) {
        typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
        const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
        return make_uint4(v.x, v.y, v.z, v.w);
    }
    return *reinterpret_cast<const uint4*>(p);
}

__device__ __forceinline__ uint4 load_or_zero(const uint16_t* p, bool valid) {
    uint4 r = make_uint4(0, 0, 0, 0);
    if (valid) r = *reinterpret_cast<const uint4*>(p);
    return r;
}

// STEP: the block first runs the QK-RMSNorm + RoPE of its query heads (and, if it owns the tile of
// the new token, of the key head, appending K and V to the cache) — the reference's separate
// launch_qk_norm_rope_cache_m1 (R17:17181) folded into the attention launch.
// GENERIC: what the decode calls of the reference's own shapes never need and therefore do not pay for — a GQA
// group served by several blocks of G heads per kv head, and the rows of one sequence as streams.
template <int G, bool STEP, bool STREAMING, bool GENERIC>
__global__ __launch_bounds__(kDecodeThreads) void decode_split_kernel(DecodeParams prm, qm_kv_cache cache) {
    request_arguments(prm, cache);
    __shared__ __attribute__((aligned(16))) uint16_t sh_qrot[STEP ? G : 1][kDim];
    __shared__ float sh_acc[kRowStreams][G][kDim];
    __shared__ float sh_m[kRowStreams][G];
    __shared__ float sh_l[kRowStreams][G];
    __shared__ int64_t sh_off[kMaxTilesPerBlock];   // element offset of each tile of this block, -1 = unreadable

    // Grid (head groups, splits, streams), x fastest: the blocks that read the eight kv heads of the same pages —
    // 32 KiB of K and 32 KiB of V that lie together in a native page — are dispatched one after the other and walk
    // their tiles side by side (ragged 64 x 256..4096: 99.1 us against 101.0 us with the split index fastest,
    // same bits).  Blocks go to the eight XCDs round-robin in that order; where the XCD would depend on the split
    // index (fewer than eight head groups) the high splits of a ragged batch are mostly empty, so the split is
    // rotated by (head group + stream) and every XCD sees every split index.
    const int split = static_cast<int>((blockIdx.x + blockIdx.y + blockIdx.z) % gridDim.y);
    const int hg = blockIdx.x;   // group of G query heads; its kv head:
    const int kvh = GENERIC ? hg / prm.head_groups_per_kv : hg;
    const int stream = blockIdx.z;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int row = lane >> 4;   // DPP row inside the wave = token slot inside a load
    const int col = lane & 15;   // 8-dim chunk

    int key_start = prm.fixed_key_start;
    int key_end = prm.fixed_key_end;
    if (prm.seq_lens) {
        key_start = 0;
        key_end = prm.seq_lens[stream];
        if (key_end > prm.max_seq_len) {
            // The grid and the workspace were sized for max_seq_len: attend what fits, flag it.
            if (tid == 0 && prm.status) atomicOr(prm.status, QM_STATUS_BAD_POSITION);
            key_end = prm.max_seq_len;
        }
    } else if (GENERIC && prm.rows_cache_before >= 0) {
        row_key_range(prm, stream, key_start, key_end);
    }
    if (key_end <= key_start) {
        // Empty context: zeros.  With several splits the merge kernel writes them.
        if (prm.max_splits == 1 && split == 0) {
            for (int o = tid; o < G * kDim; o += kDecodeThreads) {
                prm.out[(static_cast<int64_t>(stream) * prm.q_heads + hg * G) * kDim + o] = 0;
            }
        }
        return;
    }

    const int first_tile = key_start / kTile;
    const int last_tile = (key_end - 1) / kTile;
    const int tile_lo = first_tile + split * prm.tiles_per_block;
    if (tile_lo > last_tile) return;
    const int tile_hi = min(tile_lo + prm.tiles_per_block - 1, last_tile);

    // Page lookups happen once, up front, so that the streaming loop below issues nothing but
    // K/V loads to the vector memory queue (a page-table load inside the loop would make every
    // iteration wait for the whole queue to drain).
    if (tid <= tile_hi - tile_lo) {
        const int32_t* table =
            prm.page_table && !(GENERIC && prm.rows_cache_before >= 0)
                ? prm.page_table + static_cast<int64_t>(stream) * prm.pages.max_pages
                : prm.page_table;
        sh_off[tid] = tile_offset(cache, prm.pages, table, (tile_lo + tid) * kTile, kvh, prm.status);
    }

    // Query chunk of this lane for each head of the group, packed bf16 pairs.
    uint4 qv[G];
    if (STEP) {
        // Items: the G query heads; in the block that owns the new token's tile also K and V.
        // One wave per item, in the arithmetic of the append kernel (bit-identical results).
        const int position = prm.step_position;
        const bool owner = tile_lo <= position / kTile && position / kTile <= tile_hi;
        const int32_t* table = prm.page_table;
        for (int item = wave; item < G + (owner ? 2 : 0); item += kDecodeWaves) {
            if (item < G) {
                const int qh = hg * G + item;
                const HeadPair r = norm_rope_head(prm.step_q[qh * kDim + lane], prm.step_q[qh * kDim + lane + 64],
                                                  prm.step_q_norm, prm.step_cos, prm.step_sin, prm.step_epsilon, lane);
                sh_qrot[item][lane] = r.lo;
                sh_qrot[item][lane + 64] = r.hi;
                if (split == 0 && prm.step_q_rotated) {
                    prm.step_q_rotated[qh * kDim + lane] = r.lo;
                    prm.step_q_rotated[qh * kDim + lane + 64] = r.hi;
                }
            } else {
                const int64_t tile_base = tile_offset(cache, prm.pages, table, (position / kTile) * kTile, kvh,
                                                      lane == 0 ? prm.status : nullptr);
                if (tile_base >= 0) {
                    const int64_t dst = tile_base + static_cast<int64_t>(position % kTile) * kDim;
                    if (item == G) {
                        const HeadPair r = norm_rope_head(prm.step_k[kvh * kDim + lane], prm.step_k[kvh * kDim + lane + 64],
                                                          prm.step_k_norm, prm.step_cos, prm.step_sin, prm.step_epsilon, lane);
                        cache.k_pool[dst + lane] = r.lo;
                        cache.k_pool[dst + lane + 64] = r.hi;
                    } else {
                        // V is appended as it is: no norm, no rotation (R17:15515-15524).
                        cache.v_pool[dst + lane] = prm.step_v[kvh * kDim + lane];
                        cache.v_pool[dst + lane + 64] = prm.step_v[kvh * kDim + lane + 64];
                    }
                }
            }
        }
        __syncthreads();   // the appended K/V and the rotated q are visible to the whole block
#pragma unroll
        for (int g = 0; g < G; ++g) qv[g] = *reinterpret_cast<const uint4*>(&sh_qrot[g][col * 8]);
    } else {
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const int qh = hg * G + g;
            qv[g] = *reinterpret_cast<const uint4*>(
                prm.query + (static_cast<int64_t>(stream) * prm.q_heads + qh) * kDim + col * 8);
        }
    }

    float m[G], l[G], acc[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        m[g] = -INFINITY;
        l[g] = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] = 0.0f;
    }
    __syncthreads();

    // Unpredicated fetch: a token outside [key_start, key_end) is redirected to the nearest
    // token inside (same tile, so the address is valid) and its score is masked afterwards; an
    // unreadable tile reads pool offset 0 and is masked as a whole.
    uint4 kreg[4], vreg[4];
    int okmask = 0;
    auto fetch = [&](int tile, uint4* kr, uint4* vr, int& ok) {
        const int first_token = tile * kTile;
        int64_t off = sh_off[tile - tile_lo];
        const bool readable = off >= 0;
        off = readable ? off : 0;
        ok = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int token = first_token + 4 * i + row;
            const bool in_range = readable && token >= key_start && token < key_end;
            ok |= in_range ? (1 << i) : 0;
            int safe = min(max(token, key_start), key_end - 1) - first_token;
            safe = readable ? min(max(safe, 0), kTile - 1) : 0;
            const int64_t e = off + safe * kDim + col * 8;
            kr[i] = kv_load<STREAMING>(cache.k_pool + e);
            vr[i] = kv_load<STREAMING>(cache.v_pool + e);
        }
    };

    // One tile of work on a register set: scores, online softmax update, P.V.
    auto consume = [&](const uint4* kr, const uint4* vr, int ok) {
        // ---- scores of the 4 tokens this row owns, for every head of the group -------------
        float s[4][G];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int g = 0; g < G; ++g) {
                float d = 0.0f;
                d = dot2_bf16(qv[g].x, kr[i].x, d);
                d = dot2_bf16(qv[g].y, kr[i].y, d);
                d = dot2_bf16(qv[g].z, kr[i].z, d);
                d = dot2_bf16(qv[g].w, kr[i].w, d);
                d = row16_allreduce_sum(d);
                // bf16(QK) then bf16(* scale), R17:16102-16116
                d = round_bf16(round_bf16(d) * prm.scale);
                s[i][g] = (ok >> i) & 1 ? d : -INFINITY;
            }
        }
        // ---- online softmax update of this row-stream ------------------------------------------
        float p[4][G];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float mx = fmaxf(fmaxf(s[0][g], s[1][g]), fmaxf(s[2][g], s[3][g]));
            const float m_new = fmaxf(m[g], mx);
            const float m_ref = m_new == -INFINITY ? 0.0f : m_new;
            const float alpha = fast_exp2((m[g] - m_ref) * kLog2e);
            float psum = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                p[i][g] = fast_exp2((s[i][g] - m_ref) * kLog2e);
                psum += p[i][g];
            }
            l[g] = fmaf(l[g], alpha, psum);
            m[g] = m_new;
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[g][e] *= alpha;
        }
        // ---- P.V (a masked token has p = 0 and a duplicated, finite row) ---------------------------
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t w[4] = {vr[i].x, vr[i].y, vr[i].z, vr[i].w};
            const bool live = (ok >> i) & 1;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float v0 = live ? lo_bf16(w[j]) : 0.0f;
                const float v1 = live ? hi_bf16(w[j]) : 0.0f;
#pragma unroll
                for (int g = 0; g < G; ++g) {
                    acc[g][2 * j] = fmaf(p[i][g], v0, acc[g][2 * j]);
                    acc[g][2 * j + 1] = fmaf(p[i][g], v1, acc[g][2 * j + 1]);
                }
            }
        }
    };

    // Two register sets in ping-pong: the loads of one tile are in flight while the other tile
    // is consumed, with no register copies between iterations.  Every path issues exactly one
    // fetch between two consumes, so that the in-order load counter lets the consume of a set
    // start while the eight loads of the other set are still outstanding.
    uint4 kreg2[4], vreg2[4];
    int okmask2 = 0;
    int tile = tile_lo + wave;
    if (tile <= tile_hi) {
        fetch(tile, kreg, vreg, okmask);
        bool last_is_second = false;
        for (;;) {
            int next = tile + kDecodeWaves;
            if (next > tile_hi) break;
            fetch(next, kreg2, vreg2, okmask2);
            __builtin_amdgcn_sched_barrier(0);   // issue the loads before waiting on the other set
            consume(kreg, vreg, okmask);
            tile = next;
            next = tile + kDecodeWaves;
            if (next > tile_hi) {
                last_is_second = true;
                break;
            }
            fetch(next, kreg, vreg, okmask);
            __builtin_amdgcn_sched_barrier(0);
            consume(kreg2, vreg2, okmask2);
            tile = next;
        }
        if (last_is_second) {
            consume(kreg2, vreg2, okmask2);
        } else {
            consume(kreg, vreg, okmask);
        }
    }

    // ---- merge the 16 row-streams of the block -----------------------------------------------
    const int rs = wave * 4 + row;
#pragma unroll
    for (int g = 0; g < G; ++g) {
#pragma unroll
        for (int e = 0; e < 8; ++e) sh_acc[rs][g][col * 8 + e] = acc[g][e];
        if (col == 0) {
            sh_m[rs][g] = m[g];
            sh_l[rs][g] = l[g];
        }
    }
    __syncthreads();

    for (int o = tid; o < G * kDim; o += kDecodeThreads) {
        const int g = o / kDim;
        const int d = o % kDim;
        float mm = -INFINITY;
#pragma unroll
        for (int j = 0; j < kRowStreams; ++j) mm = fmaxf(mm, sh_m[j][g]);
        const float m_ref = mm == -INFINITY ? 0.0f : mm;
        float ll = 0.0f, aa = 0.0f;
#pragma unroll
        for (int j = 0; j < kRowStreams; ++j) {
            const float w = fast_exp2((sh_m[j][g] - m_ref) * kLog2e);
            ll = fmaf(sh_l[j][g], w, ll);
            aa = fmaf(sh_acc[j][g][d], w, aa);
        }
        if (prm.max_splits == 1) {
            const int qh = hg * G + g;
            prm.out[(static_cast<int64_t>(stream) * prm.q_heads + qh) * kDim + d] =
                f2bf(ll > 0.0f ? aa / ll : 0.0f);
        } else {
            float* rec = prm.partial
                + ((static_cast<int64_t>(stream) * gridDim.x + hg) * prm.max_splits + split)
                      * partial_floats<G>();
            rec[g * kDim + d] = aa;
            if (d == 0) {
                rec[G * kDim + g] = mm;
                rec[G * kDim + G + g] = ll;
            }
        }
    }
}

// Merge of the split partials of one (stream, group of G heads); also writes zeros for an empty
// context.  grid (head groups, n_streams), block G*128.
template <int G, bool GENERIC>
__global__ void decode_merge_kernel(DecodeParams prm) {
    request_arguments(prm);
    const int hg = blockIdx.x;
    const int stream = blockIdx.y;
    const int g = threadIdx.x / kDim;
    const int d = threadIdx.x % kDim;
    const int qh = hg * G + g;
    uint16_t* dst = prm.out + (static_cast<int64_t>(stream) * prm.q_heads + qh) * kDim + d;

    const float* base = prm.partial
        + (static_cast<int64_t>(stream) * gridDim.x + hg) * prm.max_splits * partial_floats<G>();

    // All loads of a round — the context length, the statistics of up to kMergeRound splits and
    // this thread's accumulator column of each — are issued before anything is consumed, so the
    // kernel pays one memory latency per round.  Records of splits that do not exist hold
    // stale workspace contents; they are read (the addresses are valid) and then ignored.
    __shared__ float sh_w[kMergeRound][G];
    __shared__ float sh_l[kMergeRound][G];
    float ll = 0.0f, aa = 0.0f;
    float m_run = -INFINITY;
    int splits = 0;
    for (int s0 = 0; s0 < prm.max_splits; s0 += kMergeRound) {
        const int cap = min(prm.max_splits - s0, kMergeRound);
        float stat_m = 0.0f, stat_l = 0.0f;
        if (static_cast<int>(threadIdx.x) < cap * G) {
            const float* rec = base + static_cast<int64_t>(s0 + threadIdx.x / G) * partial_floats<G>();
            stat_m = rec[G * kDim + threadIdx.x % G];
            stat_l = rec[G * kDim + G + threadIdx.x % G];
        }
        float part[kMergeRound];
#pragma unroll
        for (int u = 0; u < kMergeRound; ++u) {
            part[u] = u < cap ? base[static_cast<int64_t>(s0 + u) * partial_floats<G>() + g * kDim + d] : 0.0f;
        }
        if (s0 == 0) {
            int key_start = prm.fixed_key_start;
            int key_end = prm.fixed_key_end;
            if (prm.seq_lens) {
                key_start = 0;
                key_end = min(prm.seq_lens[stream], prm.max_seq_len);
            } else if (GENERIC && prm.rows_cache_before >= 0) {
                row_key_range(prm, stream, key_start, key_end);
            }
            if (key_end <= key_start) {
                *dst = 0;
                return;
            }
            const int tiles = (key_end - 1) / kTile - key_start / kTile + 1;
            splits = min((tiles + prm.tiles_per_block - 1) / prm.tiles_per_block, prm.max_splits);
        }
        const int n = min(splits - s0, cap);
        if (n <= 0) break;
        __syncthreads();
        if (static_cast<int>(threadIdx.x) < cap * G) {
            sh_w[threadIdx.x / G][threadIdx.x % G] = stat_m;
            sh_l[threadIdx.x / G][threadIdx.x % G] = stat_l;
        }
        __syncthreads();
        float mm = m_run;
        for (int s = 0; s < n; ++s) mm = fmaxf(mm, sh_w[s][g]);
        const float m_ref = mm == -INFINITY ? 0.0f : mm;
        const float rescale = fast_exp2((m_run - m_ref) * kLog2e);
        ll *= rescale;
        aa *= rescale;
        m_run = mm;
#pragma unroll
        for (int u = 0; u < kMergeRound; ++u) {
            if (u < n) {
                const float w = fast_exp2((sh_w[u][g] - m_ref) * kLog2e);
                ll = fmaf(sh_l[u][g], w, ll);
                aa = fmaf(part[u], w, aa);
            }
        }
    }
    *dst = f2bf(ll > 0.0f ? aa / ll : 0.0f);
}

// ---- host side -------------------------------------------------------------------------------

// Split plan shared by the workspace query and the launch: pure function of the shape.
struct DecodePlan {
    int tiles_per_block;
    int max_splits;
    int splits_bound;            // what the workspace is sized for (>= max_splits)
};

inline DecodePlan plan_decode(int n_streams, int kv_heads, int max_seq_len) {
    const int64_t max_tiles = (static_cast<int64_t>(max_seq_len) + kTile - 1) / kTile + 1;
    int tiles_per_block = option_value(QM_OPT_DECODE_TILES_PER_BLOCK);
    if (tiles_per_block <= 0) {
        // One tile per wave at least; a block should not be shorter than it has to be (its set-up,
        // the merge of its 16 row-streams and its partial record are fixed costs), yet the grid
        // must keep a few thousand blocks so that ragged lengths balance: about 8 blocks per CU,
        // at most 24 tiles (384 tokens, 192 KiB of K+V) per block.  Ragged 64 x 256..4096, three
        // seeds: 4 tiles 126 / 132 / 111 us, 8: 106 / 113 / 93, 16: 101 / 97 / 88, 24: 100 / 96 / 88,
        // 32: 100 / 95 / 87, 48: 102 / 99 / 89.
        const int64_t total = max_tiles * n_streams * kv_heads;
        int64_t t = total / (256 * 8);
        t = (t + 3) / 4 * 4;
        if (t < 4) t = 4;
        if (t > 24) t = 24;
        // The merge kernel takes the records of kMergeRound splits per memory round trip: a stream is not
        // cut into more than that while blocks may still grow (one stream at context 2048 is 129 tiles:
        // 33 splits of 4 tiles 9.9 us per fused step, 17 splits of 8 tiles 8.8 us, 9 of 16 10.1 us).
        const int64_t for_one_round = ((max_tiles + kMergeRound - 1) / kMergeRound + 3) / 4 * 4;
        if (t < for_one_round) t = for_one_round;
        tiles_per_block = static_cast<int>(t < kMaxTilesPerBlock ? t : kMaxTilesPerBlock);
    }
    if (tiles_per_block > kMaxTilesPerBlock) tiles_per_block = kMaxTilesPerBlock;
    DecodePlan plan;
    plan.tiles_per_block = tiles_per_block;
    plan.max_splits = static_cast<int>((max_tiles + tiles_per_block - 1) / tiles_per_block);
    // What the workspace is sized for: a bound on max_splits that never shrinks as the context grows (the
    // automatic choice above steps to longer blocks), so that a workspace sized for the longest context serves
    // every shorter one.
    plan.splits_bound = plan.max_splits;
    if (option_value(QM_OPT_DECODE_TILES_PER_BLOCK) <= 0) {
        const int64_t short_blocks = std::min<int64_t>((max_tiles + 3) / 4, kMergeRound);
        const int64_t long_contexts = (max_tiles + kMaxTilesPerBlock - 1) / kMaxTilesPerBlock;
        plan.splits_bound = static_cast<int>(std::max(short_blocks, long_contexts));
    }
    return plan;
}

inline size_t decode_workspace_bytes(int n_streams, int q_heads, int kv_heads, int max_seq_len) {
    const DecodePlan plan = plan_decode(n_streams, kv_heads, max_seq_len);
    if (plan.splits_bound <= 1) return 0;
    const int g = q_heads / kv_heads;
    return static_cast<size_t>(n_streams) * kv_heads * plan.splits_bound * (g * kDim + 2 * g)
         * sizeof(float);
}

template <int G, bool STREAMING>
int32_t launch_split(const DecodeParams& prm, const qm_kv_cache& cache, int n_streams, bool generic, hipStream_t stream) {
    const dim3 grid(cache.kv_heads * prm.head_groups_per_kv, prm.max_splits, n_streams);
    if (prm.step_q) {
        if (generic) return QM_ERR_GEOMETRY;   // the fused step is built for groups of 1, 2 and 4 heads
        hipLaunchKernelGGL((decode_split_kernel<G, true, STREAMING, false>), grid, dim3(kDecodeThreads), 0, stream, prm, cache);
    } else if (generic) {
        hipLaunchKernelGGL((decode_split_kernel<G, false, STREAMING, true>), grid, dim3(kDecodeThreads), 0, stream, prm, cache);
    } else {
        hipLaunchKernelGGL((decode_split_kernel<G, false, STREAMING, false>), grid, dim3(kDecodeThreads), 0, stream, prm, cache);
    }
    return launch_status();
}

template <int G>
int32_t launch_decode(const DecodeParams& prm, const qm_kv_cache& cache, int n_streams, bool streaming,
                      hipStream_t stream, bool merge) {
    const bool generic = prm.head_groups_per_kv > 1 || prm.rows_cache_before >= 0;
    int32_t rc = streaming ? launch_split<G, true>(prm, cache, n_streams, generic, stream)
                           : launch_split<G, false>(prm, cache, n_streams, generic, stream);
    if (rc != QM_OK) return rc;
    if (merge && prm.max_splits > 1) {
        const dim3 grid(cache.kv_heads * prm.head_groups_per_kv, n_streams);
        if (generic) hipLaunchKernelGGL((decode_merge_kernel<G, true>), grid, dim3(G * kDim), 0, stream, prm);
        else hipLaunchKernelGGL((decode_merge_kernel<G, false>), grid, dim3(G * kDim), 0, stream, prm);
        rc = launch_status();
    }
    return rc;
}

// Rows of one sequence as streams: what qm_attention_rows adds to a call.
struct RowsOfOneSequence {
    int cache_before;
    int sliding_window;
};

int32_t decode_common(const uint16_t* query, const qm_kv_cache* cache, const int32_t* page_table,
                      int32_t max_pages, const int32_t* seq_lens, int32_t n_streams,
                      int32_t key_start, int32_t key_end, int32_t max_seq_len, uint16_t* out,
                      int32_t q_heads, float scale, void* workspace, size_t workspace_bytes,
                      uint32_t* status_dev, void* hip_stream, const DecodeParams* step = nullptr,
                      const RowsOfOneSequence* rows = nullptr, DecodeSplitInfo* unmerged = nullptr) {
    if ((!query && !step) || !out) return QM_ERR_NULL;
    int32_t rc = check_cache(cache, max_pages);
    if (rc != QM_OK) return rc;
    rc = check_group(q_heads, cache->kv_heads);
    if (rc != QM_OK) return rc;
    if ((reinterpret_cast<uintptr_t>(query) & 15)) return QM_ERR_GEOMETRY;
    if (n_streams < 0 || n_streams > 65535 || q_heads > 65535) return QM_ERR_ARGUMENT;
    if (max_seq_len < 0) return QM_ERR_ARGUMENT;
    if (max_seq_len > cache_capacity(cache, max_pages)) return QM_ERR_SLOT_RANGE;
    const int loads = option_value(QM_OPT_DECODE_STREAMING_LOADS);
    if (loads < 0 || loads > 2) return QM_ERR_ARGUMENT;
    if (n_streams == 0) return QM_OK;

    const DecodePlan plan = plan_decode(n_streams, cache->kv_heads, max_seq_len);
    if (plan.max_splits > 65535) return QM_ERR_ARGUMENT;     // (a grid dimension)
    const size_t need = decode_workspace_bytes(n_streams, q_heads, cache->kv_heads, max_seq_len);
    if (need > 0 && (!workspace || workspace_bytes < need)) return QM_ERR_WORKSPACE;
    if (need > 0 && (reinterpret_cast<uintptr_t>(workspace) & 3)) return QM_ERR_WORKSPACE;

    DecodeParams prm;
    prm.query = query;
    prm.out = out;
    prm.page_table = page_table;
    prm.seq_lens = seq_lens;
    prm.partial = static_cast<float*>(workspace);
    prm.status = status_dev;
    prm.pages = make_page_map(cache->page_size, max_pages);
    prm.max_seq_len = max_seq_len;
    prm.fixed_key_start = key_start;
    prm.fixed_key_end = key_end;
    prm.tiles_per_block = plan.tiles_per_block;
    prm.max_splits = plan.max_splits;
    prm.q_heads = q_heads;
    prm.scale = scale;
    // Heads per block: the largest instantiated G that divides the GQA group.
    const int group = q_heads / cache->kv_heads;
    const int heads_per_block = group % 4 == 0 ? 4 : group % 2 == 0 ? 2 : 1;
    prm.head_groups_per_kv = group / heads_per_block;
    prm.rows_cache_before = rows ? rows->cache_before : -1;
    prm.rows_window = rows ? rows->sliding_window : 0;
    prm.step_q = nullptr;
    if (step) {
        prm.step_q = step->step_q; prm.step_k = step->step_k; prm.step_v = step->step_v;
        prm.step_q_norm = step->step_q_norm; prm.step_k_norm = step->step_k_norm;
        prm.step_cos = step->step_cos; prm.step_sin = step->step_sin;
        prm.step_q_rotated = step->step_q_rotated;
        prm.step_position = step->step_position; prm.step_epsilon = step->step_epsilon;
    }

    // Upper bound of the K and V bytes one call reads.
    const int64_t context_bytes = (rows ? 1 : static_cast<int64_t>(n_streams)) * (seq_lens || rows ? max_seq_len : key_end - key_start)
                                * cache->kv_heads * kDim * 2 * 2;
    bool streaming = context_bytes > kStreamingContextBytes;
    if (loads == 1) streaming = false;
    if (loads == 2) streaming = true;

    hipStream_t s = static_cast<hipStream_t>(hip_stream);
    // The caller combines the records itself (one stream) if one round of the merge holds them; a context so long that
    // it does not is merged here as always and handed over as if it had been a single split.
    const bool leave_unmerged = unmerged && plan.max_splits > 1 && plan.max_splits <= kMergeRound;
    if (unmerged) {
        const int tiles = key_end > key_start ? (key_end - 1) / kTile - key_start / kTile + 1 : 0;
        unmerged->max_splits = plan.max_splits;
        unmerged->splits = std::min((tiles + plan.tiles_per_block - 1) / plan.tiles_per_block, plan.max_splits);   // as the merge kernel counts them
        unmerged->records = leave_unmerged ? static_cast<const float*>(workspace) : nullptr;
    }
    switch (heads_per_block) {
        case 1: return launch_decode<1>(prm, *cache, n_streams, streaming, s, !leave_unmerged);
        case 2: return launch_decode<2>(prm, *cache, n_streams, streaming, s, !leave_unmerged);
        case 4: return launch_decode<4>(prm, *cache, n_streams, streaming, s, !leave_unmerged);
    }
    return QM_ERR_GEOMETRY;
}

// ---- split records in library-owned device memory --------------------------------------------
// qm_decode_attention_ragged_static keeps the split records in this array instead of a caller's
// workspace.  Every GPU the library runs on holds its own copy at its own address until the
// process ends.  In host code the array's name is only a handle for hipGetSymbolAddress: kernels
// are given the address that call returns for the current device, never the name.
constexpr size_t kStaticScratchBytes = QM_DECODE_STATIC_SCRATCH_BYTES;
static __device__ __attribute__((used)) __align__(256) unsigned char scratch[kStaticScratchBytes];

// Device address of `scratch` on the current device, looked up once per device.
int32_t static_scratch_address(void** address) {
    static std::atomic<void*> known[kMaxDevices];
    int dev = 0;
    const hipError_t e0 = hipGetDevice(&dev);
    if (e0 != hipSuccess) return hip_code(e0);
    if (dev < 0 || dev >= kMaxDevices) return QM_ERR_NO_DEVICE;
    void* ptr = known[dev].load(std::memory_order_acquire);
    if (!ptr) {
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return hip_code(e);
        if (!ptr) return QM_ERR_NO_DEVICE;
        known[dev].store(ptr, std::memory_order_release);
    }
    *address = ptr;
    return QM_OK;
}

}  // namespace qm

extern "C" size_t qm_decode_workspace_bytes(int32_t n_streams, int32_t q_heads, int32_t kv_heads,
                                            int32_t max_seq_len) {
    if (n_streams <= 0 || q_heads <= 0 || kv_heads <= 0 || max_seq_len < 0 || q_heads % kv_heads)
        return 0;
    return qm::decode_workspace_bytes(n_streams, q_heads, kv_heads, max_seq_len);
}

extern "C" int32_t qm_decode_attention(
    const uint16_t* query,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    uint16_t* context_out,
    int32_t q_heads, int32_t cache_before, int32_t sliding_window, float scale,
    void* workspace, size_t workspace_bytes, void* hip_stream) {
    if (cache_before < 0) return QM_ERR_ARGUMENT;
    // Key range of R17:16032-16036.
    const int32_t key_end = cache_before + 1;
    const int32_t window_start = key_end - sliding_window;
    const int32_t key_start = sliding_window > 0 ? (window_start > 0 ? window_start : 0) : 0;
    if (cache && !page_table && max_pages > 0 && cache->page_size > 0
        && cache_before / cache->page_size >= cache->n_pages)
        return QM_ERR_SLOT_RANGE;
    return qm::decode_common(query, cache, page_table, max_pages, nullptr, 1, key_start, key_end,
                             key_end, context_out, q_heads, scale, workspace, workspace_bytes,
                             nullptr, hip_stream);
}

extern "C" int32_t qm_decode_attention_ragged(
    const uint16_t* query,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    const int32_t* seq_lens, int32_t n_streams, int32_t max_seq_len,
    uint16_t* context_out,
    int32_t q_heads, float scale,
    void* workspace, size_t workspace_bytes, uint32_t* status_dev, void* hip_stream) {
    if (!seq_lens || !page_table) return QM_ERR_NULL;
    return qm::decode_common(query, cache, page_table, max_pages, seq_lens, n_streams, 0, 0,
                             max_seq_len, context_out, q_heads, scale, workspace, workspace_bytes,
                             status_dev, hip_stream);
}

namespace qm {

int32_t decode_step(
    const uint16_t* q, const uint16_t* k, const uint16_t* v,
    const uint16_t* q_norm_w, const uint16_t* k_norm_w,
    const uint16_t* cos_row, const uint16_t* sin_row,
    uint16_t* q_rotated_out,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    uint16_t* context_out,
    int32_t q_heads, int32_t position, int32_t sliding_window, float scale, float epsilon,
    void* workspace, size_t workspace_bytes, uint32_t* status_dev, void* hip_stream, DecodeSplitInfo* unmerged) {
    if (!q || !k || !v || !q_norm_w || !k_norm_w || !cos_row || !sin_row) return QM_ERR_NULL;
    if (position < 0) return QM_ERR_SLOT_RANGE;
    const int32_t key_end = position + 1;
    const int32_t window_start = key_end - sliding_window;
    const int32_t key_start = sliding_window > 0 ? (window_start > 0 ? window_start : 0) : 0;
    if (cache && max_pages > 0 && cache->page_size > 0) {
        if (position / cache->page_size >= max_pages) return QM_ERR_SLOT_RANGE;
        if (!page_table && position / cache->page_size >= cache->n_pages) return QM_ERR_SLOT_RANGE;
    }
    DecodeParams step = {};
    step.step_q = q; step.step_k = k; step.step_v = v;
    step.step_q_norm = q_norm_w; step.step_k_norm = k_norm_w;
    step.step_cos = cos_row; step.step_sin = sin_row;
    step.step_q_rotated = q_rotated_out;
    step.step_position = position; step.step_epsilon = epsilon;
    return decode_common(nullptr, cache, page_table, max_pages, nullptr, 1, key_start, key_end, key_end,
                         context_out, q_heads, scale, workspace, workspace_bytes, status_dev, hip_stream, &step, nullptr, unmerged);
}

}  // namespace qm

extern "C" int32_t qm_decode_step_fused(
    const uint16_t* q, const uint16_t* k, const uint16_t* v,
    const uint16_t* q_norm_w, const uint16_t* k_norm_w,
    const uint16_t* cos_row, const uint16_t* sin_row,
    uint16_t* q_rotated_out,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    uint16_t* context_out,
    int32_t q_heads, int32_t position, int32_t sliding_window, float scale, float epsilon,
    void* workspace, size_t workspace_bytes, uint32_t* status_dev, void* hip_stream) {
    return qm::decode_step(q, k, v, q_norm_w, k_norm_w, cos_row, sin_row, q_rotated_out, cache, page_table, max_pages, context_out,
                           q_heads, position, sliding_window, scale, epsilon, workspace, workspace_bytes, status_dev, hip_stream,
                           nullptr);
}

extern "C" size_t qm_attention_rows_workspace_bytes(int32_t query_length, int32_t q_heads, int32_t kv_heads,
                                                    int32_t key_end) {
    return qm_decode_workspace_bytes(query_length, q_heads, kv_heads, key_end);
}

extern "C" int32_t qm_attention_rows(
    const uint16_t* query,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    uint16_t* context_out,
    int32_t query_length, int32_t cache_before, int32_t q_heads, int32_t sliding_window, float scale,
    void* workspace, size_t workspace_bytes, uint32_t* status_dev, void* hip_stream) {
    if (query_length < 0 || cache_before < 0) return QM_ERR_ARGUMENT;
    if (static_cast<int64_t>(cache_before) + query_length > INT32_MAX) return QM_ERR_SLOT_RANGE;
    const int32_t key_end = cache_before + query_length;   // of the last row
    if (cache && !page_table && max_pages > 0 && cache->page_size > 0 && query_length > 0
        && (key_end - 1) / cache->page_size >= cache->n_pages)
        return QM_ERR_SLOT_RANGE;
    const qm::RowsOfOneSequence rows = {cache_before, sliding_window};
    return qm::decode_common(query, cache, page_table, max_pages, nullptr, query_length, 0, 0, key_end,
                             context_out, q_heads, scale, workspace, workspace_bytes, status_dev, hip_stream,
                             nullptr, &rows);
}

extern "C" int32_t qm_decode_attention_ragged_static(
    const uint16_t* query,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    const int32_t* seq_lens, int32_t n_streams, int32_t max_seq_len,
    uint16_t* context_out,
    int32_t q_heads, float scale, uint32_t* status_dev, void* hip_stream) {
    if (!seq_lens || !page_table) return QM_ERR_NULL;
    if (cache && n_streams > 0 && q_heads > 0 && cache->kv_heads > 0 && q_heads % cache->kv_heads == 0 && max_seq_len >= 0
        && qm::decode_workspace_bytes(n_streams, q_heads, cache->kv_heads, max_seq_len) > qm::kStaticScratchBytes)
        return QM_ERR_WORKSPACE;   // the shape needs more split records than the array holds
    void* records = nullptr;
    const int32_t rc = qm::static_scratch_address(&records);
    if (rc != QM_OK) return rc;
    // Nothing in the array has to start at zero: records of splits that do not exist are never used.
    return qm::decode_common(query, cache, page_table, max_pages, seq_lens, n_streams, 0, 0,
                             max_seq_len, context_out, q_heads, scale, records, qm::kStaticScratchBytes,
                             status_dev, hip_stream);
}
