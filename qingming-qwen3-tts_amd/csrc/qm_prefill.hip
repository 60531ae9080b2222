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
// Two kernels share this file and give the same bits: the uniform waves described here (the
// compiler's order inside a wave: all MFMAs of a product, then all of the softmax arithmetic) and
// the interleaved waves, which alternate MFMAs and softmax arithmetic instruction by instruction
// and are the ones the host launches by default; their comments say what was measured.  (A third
// design, blocks of four matrix waves paired with four softmax waves that hand the 32 x 32 chunks
// over through LDS, gave the same bits at 37.7 us / 398 us for 4 x 1024 / 4 x 4096 tokens against
// 30.5 / 316 for the interleaved waves: with phases of eight MFMAs and about 150 VALU instructions
// the two kinds of work mostly took turns on a SIMD whoever issued them.  It is no longer part of
// this file.)  This kernel stays within 256 registers and
// 72 KB of LDS so that two blocks share a CU and fill each other's waits.
// Variants of it that were measured and dropped (batch 4 x 1024 tokens / 4 x 4096 tokens, this
// one: 42 us / 381 us): three LDS stages with 316 registers, one wave per SIMD (51 us / 467 us);
// eight-wave blocks whose two wave groups split each key tile and merge through LDS (41 us /
// 421 us: the longest block is halved, but the groups meet at a barrier per tile and run in step).
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
// Causality.  A key after a query row never contributes, whatever it holds; keys of later 16-row groups are not
// read into the product at all.  Inside a 16-key group that the mask cuts the mask is P = 0 times V; such a group is
// checked for non-finite V values, which are then taken out of the matrix product and added for the rows that see
// them (add_non_finite_products), so that 0 x inf never forms.
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
    int heavy_groups;            // (interleaved kernel) leading groups of blocks, heaviest query tile first; the rest ascend
    int dealt_pages;             // (interleaved kernel) the whole grid is resident at once: the light blocks write the heavy blocks' pages
    // (interleaved kernel, key split) a query tile of n key tiles is shared by min(ceil(n / split_chunk), 3) blocks
    int split_chunk;             // 0: no query tile is split
    int split_slots;             // query tiles per pair that are split (the last ones)
    float* split_partials;       // [pair][split query tile][part][kSplitRecordFloats]
    int* split_tickets;          // [pair][split query tile][8]: (epoch << 4 | arrivals), then per part the epoch of its published record
    int split_epoch;             // 1 .. 2^27 - 1, another value for every launch that splits
    float scale;
    // (chunk kernel) the rows continue a sequence: row i stands at position cache_before + i and attends keys
    // 0 .. cache_before + i of the key_count = cache_before + seq keys that k and v hold
    int cache_before;
    int key_count;
    // (chunk kernel, key split) the key tiles of a query tile go to blocks in runs of chunk_run; a query tile of more
    // than one run leaves a record per run and prefill_chunk_merge_kernel combines them
    int chunk_parts;             // blocks per (pair, query tile) in the grid; 1: no split
    int chunk_run;
    float* chunk_records;        // [pair][query tile][part][kChunkRecordFloats]
    // (chunk kernel) keys and values are read from a paged cache: page ids of batch entry b at chunk_table +
    // b * pages.max_pages, the pool described by the kernel's qm_kv_cache argument; k and v are then unused
    const int32_t* chunk_table;
    int chunk_paged;
};

constexpr int kChunkRecordFloats = 66 * kPfThreads;   // per thread: 64 of O (unnormalised), the reference maximum, the sum

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

// ---- strict causality inside a 16-key group that the mask cuts ----------------------------------------------------
// The mask is P = 0, and the MFMA still multiplies the masked key's V by it: 0 x (inf or NaN) is NaN, so a non-finite V
// of a key after a query row would reach that row, which the reference never lets happen (it does not touch keys after
// the row, R17:15784-15789).  Only a group the mask cuts for some column of the wave is concerned (groups wholly
// visible are multiplied as the reference multiplies them, groups wholly masked are skipped), and only if it holds a
// non-finite V at all, which costs three instructions per fragment register to find out.  Then the fragments'
// non-finite elements are set to zero, so that the MFMA adds the finite products only, and the products of the
// non-finite elements are added one by one, for the columns that see the key: fmaf(p, v, o) as the reference forms
// it (p = 0 included: a probability that underflowed gives NaN there too).

// Whether any lane of the wave holds a non-finite bf16 in the four fragments (a half whose exponent bits are all ones
// carries into bit 15 / 31).
__device__ __forceinline__ uint32_t exponent_carries(const bf16x8_t& f) {
    const uint4 w = __builtin_bit_cast(uint4, f);
    return ((w.x & 0x7f807f80u) + 0x00800080u) | ((w.y & 0x7f807f80u) + 0x00800080u)
         | ((w.z & 0x7f807f80u) + 0x00800080u) | ((w.w & 0x7f807f80u) + 0x00800080u);
}
__device__ __forceinline__ bool any_non_finite(const bf16x8_t& f0, const bf16x8_t& f1, const bf16x8_t& f2, const bf16x8_t& f3) {
    const uint32_t acc = exponent_carries(f0) | exponent_carries(f1) | exponent_carries(f2) | exponent_carries(f3);
    return __builtin_amdgcn_ballot_w64((acc & 0x80008000u) != 0) != 0;
}
__device__ __forceinline__ uint32_t finite_halves(uint32_t x) {
    const uint32_t t = (x & 0x7f807f80u) + 0x00800080u;
    return x & ((t & 0x8000u ? 0u : 0xffffu) | (t & 0x80000000u ? 0u : 0xffff0000u));
}
__device__ __forceinline__ void zero_non_finite(bf16x8_t& f) {
    uint4 w = __builtin_bit_cast(uint4, f);
    w.x = finite_halves(w.x); w.y = finite_halves(w.y); w.z = finite_halves(w.z); w.w = finite_halves(w.w);
    f = __builtin_bit_cast(bf16x8_t, w);
}
// The products of the non-finite V elements of the 16 keys key0 .. key0 + 15, for the columns that see the key.
// p_hi (+ p_lo): this lane's eight probabilities of the group as the MFMA takes them (element i = key
// 8 (i / 4) + 4 grp + i % 4 of the group; the lane of the other half of the wave holds the other eight).
// v_group: the V row of key key0 (the rows of the group follow at stride_token elements); a lane's accumulators
// o[dt][4 rq + c] are dims 32 dt + 8 rq + 4 grp + c.
template <bool TWO_PARTS>
__device__ __forceinline__ void add_non_finite_products(f32x16_t (&o)[4], uint4 p_hi, uint4 p_lo, const uint16_t* v_group,
                                                        int64_t stride_token, int key0, int key_count, int my_pos, int grp) {
#pragma unroll 1
    for (int jj = 0; jj < 16; ++jj) {
        const int key = key0 + jj;
        if (key >= key_count) break;
        const int owner = (jj >> 2) & 1;                   // the half of the wave that holds this key's probability
        const int i = 4 * (jj >> 3) + (jj & 3);
        const int w = i >> 1;
        const uint32_t word_hi = w == 0 ? p_hi.x : w == 1 ? p_hi.y : w == 2 ? p_hi.z : p_hi.w;
        float mine = (i & 1) ? hi_bf16(word_hi) : lo_bf16(word_hi);
        if (TWO_PARTS) {
            const uint32_t word_lo = w == 0 ? p_lo.x : w == 1 ? p_lo.y : w == 2 ? p_lo.z : p_lo.w;
            mine += (i & 1) ? hi_bf16(word_lo) : lo_bf16(word_lo);
        }
        const auto both = __builtin_amdgcn_permlane32_swap(__float_as_uint(mine), __float_as_uint(mine), false, false);
        // (after the swap the first word is the lower half's value in both halves, the second the upper half's)
        const float prob = __uint_as_float(owner == 0 ? both[0] : both[1]);
        if (key > my_pos) continue;                        // this column does not see the key (per lane)
        const uint16_t* row = v_group + static_cast<int64_t>(jj) * stride_token + 4 * grp;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) {
#pragma unroll
            for (int rq = 0; rq < 4; ++rq) {
                // (one request at a time: this path is taken for non-finite inputs only and must not cost the
                // kernel registers)
                __builtin_amdgcn_sched_barrier(0);
                const uint2 four = *reinterpret_cast<const uint2*>(row + 32 * dt + 8 * rq);
                const float v0 = lo_bf16(four.x), v1 = hi_bf16(four.x), v2 = lo_bf16(four.y), v3 = hi_bf16(four.y);
                if (!(fabsf(v0) <= 3.3895314e38f)) o[dt][4 * rq + 0] = fmaf(prob, v0, o[dt][4 * rq + 0]);
                if (!(fabsf(v1) <= 3.3895314e38f)) o[dt][4 * rq + 1] = fmaf(prob, v1, o[dt][4 * rq + 1]);
                if (!(fabsf(v2) <= 3.3895314e38f)) o[dt][4 * rq + 2] = fmaf(prob, v2, o[dt][4 * rq + 2]);
                if (!(fabsf(v3) <= 3.3895314e38f)) o[dt][4 * rq + 3] = fmaf(prob, v3, o[dt][4 * rq + 3]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
}

template <int N> using int_c = std::integral_constant<int, N>;
template <bool B> using bool_c = std::integral_constant<bool, B>;

// CHUNK: the query rows stand at positions cache_before + row (prefill_chunk_kernel); otherwise at their row.
// G: query heads per kv head (the GQA group; 1, 2 or 4).  A wave's 32 MFMA columns are 32 / G query rows x G heads,
// so every K and V fragment serves all G heads, and a block is 4 x 32 / G query rows.  The whole-prompt kernels are
// built for G = 2 only (their query tiles are as long as a key tile); the chunk kernel for 1, 2 and 4.
template <bool PRECISE, bool ROUND, bool CHUNK = false, int G = 2>
__device__ __forceinline__ void prefill_body(const PrefillParams& prm, const qm_kv_cache& cache,
                                             unsigned char* pf_smem, int qt, int pair, int part = 0) {
    static_assert(G == 1 || G == 2 || G == 4, "the GQA group the MFMA columns are dealt for");
    static_assert(CHUNK || G == 2, "the whole-prompt kernels index key tiles by query tiles of the same length");
    constexpr int R = 32 / G;            // query rows of a wave
    constexpr int BM = 4 * R;            // query rows of a block
    PfStage* st = reinterpret_cast<PfStage*>(pf_smem);

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int col = lane & 31;       // MFMA column = (query row % 16, head)
    const int grp = lane >> 5;       // MFMA k / row group

    const int b = pair / prm.kv_heads;
    const int kvh = pair % prm.kv_heads;
    const int S = prm.seq;
    const int SK = CHUNK ? prm.key_count : S;        // keys that k and v hold
    const int shift = CHUNK ? prm.cache_before : 0;  // position of query row 0
    const int q_heads = G * prm.kv_heads;

    const int q0 = qt * BM;
    const int my_row = q0 + R * wave + (col % R);     // query row of this lane's column
    const int my_pos = my_row + shift;                // the last key it attends
    const int my_head = G * kvh + col / R;
    const int wave_last_row = q0 + R * wave + R - 1 + shift;   // as a position

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
    // (chunk kernel over a paged cache) where key `key` of this (batch, kv head) lies in the pool: its page's entry of
    // the batch entry's table, then page, head and token strides.  An entry outside the pool is flagged and read as
    // page 0, so that nothing outside the pool is touched.
    uint32_t chunk_page_err = 0;
    auto paged_offset = [&](int key) -> int64_t {
        const int page = page_of(prm.pages, key);
        int phys = prm.chunk_table[static_cast<int64_t>(b) * prm.pages.max_pages + page];
        if (phys < 0 || phys >= cache.n_pages) {
            chunk_page_err |= QM_STATUS_BAD_PAGE;
            phys = 0;
        }
        return static_cast<int64_t>(phys) * cache.stride_page + static_cast<int64_t>(kvh) * cache.stride_head
             + static_cast<int64_t>(key - page * prm.pages.page_size) * kDim;
    };
    // The four 16-key groups of a 64-key tile lie in four pages at most (a page holds a multiple of 16 keys), and
    // which pages is the same for every lane: four table entries per tile, asked for a tile ahead so that the tile's
    // own loads do not wait for them.  (A group at or beyond the keys there are names the page of the last key.)
    int ne0 = 0, ne1 = 0, ne2 = 0, ne3 = 0, ne_tile = -1;
    auto group_page = [&](int key) -> int { return page_of(prm.pages, min(key, SK - 1)); };
    auto fetch_tile_entries = [&](int tile) {
        const int32_t* tab = prm.chunk_table + static_cast<int64_t>(b) * prm.pages.max_pages;
        ne0 = tab[group_page(tile * kBN)];
        ne1 = tab[group_page(tile * kBN + 16)];
        ne2 = tab[group_page(tile * kBN + 32)];
        ne3 = tab[group_page(tile * kBN + 48)];
        ne_tile = tile;
    };
    auto checked_entry = [&](int phys) -> int {
        if (phys < 0 || phys >= cache.n_pages) {
            chunk_page_err |= QM_STATUS_BAD_PAGE;
            phys = 0;
        }
        return phys;
    };
    auto load_tile = [&](int tile) {
        const int key0 = tile * kBN;
        if (CHUNK && prm.chunk_paged) {
            if (ne_tile != tile) fetch_tile_entries(tile);
            const int e0 = checked_entry(ne0), e1 = checked_entry(ne1), e2 = checked_entry(ne2), e3 = checked_entry(ne3);
            const int64_t head_off = static_cast<int64_t>(kvh) * cache.stride_head;
            // (a key at or beyond the keys there are is redirected to the last key, as below)
            const int vg = v_kg >> 2;                       // the 16-key group of this lane's four V rows
            const int ve = vg == 0 ? e0 : vg == 1 ? e1 : vg == 2 ? e2 : e3;
            const int v_first = group_page(key0 + 16 * vg) * prm.pages.page_size;
            const uint16_t* v_page = cache.v_pool + (static_cast<int64_t>(ve) * cache.stride_page + head_off) + 8 * v_dc;
            each_stage([&](uint4& kk, uint4& vv, int i) {
                const int e = i == 0 ? e0 : i == 1 ? e1 : i == 2 ? e2 : e3;
                const int key = min(key0 + (tid >> 4) + 16 * i, SK - 1);
                const int k_first = group_page(key0 + 16 * i) * prm.pages.page_size;
                kk = *reinterpret_cast<const uint4*>(cache.k_pool + (static_cast<int64_t>(e) * cache.stride_page + head_off)
                                                     + (key - k_first) * kDim + 8 * (tid & 15));
                const int vkey = min(key0 + 4 * v_kg + i, SK - 1);
                vv = *reinterpret_cast<const uint4*>(v_page + (vkey - v_first) * kDim);
            });
            fetch_tile_entries(tile + 1);
        } else if (key0 + kBN <= SK) {
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
                const int key = min(key0 + (tid >> 4) + 16 * i, SK - 1);
                kk = *reinterpret_cast<const uint4*>(k_src + static_cast<uint32_t>(key * kv_row32));
                const int vkey = min(key0 + 4 * v_kg + i, SK - 1);
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
            bf16x8_t v0 = vf[4 * kg], v1 = vf[4 * kg + 1], v2 = vf[4 * kg + 2], v3 = vf[4 * kg + 3];
            // (a group the mask cuts for some column of the wave — its last key lies after the wave's first row, or
            // beyond the keys there are — with a non-finite V: see add_non_finite_products)
            if (decltype(diag)::value && (key_base + 16 * kg + 15 > wave_last_row - (R - 1) || key_base + 16 * kg + 15 >= SK)
                && any_non_finite(v0, v1, v2, v3)) {
                zero_non_finite(v0); zero_non_finite(v1); zero_non_finite(v2); zero_non_finite(v3);
                // (a paged cache: the group's sixteen keys lie in one page, pages being multiples of sixteen tokens)
                const int group_key = key_base + 16 * kg;
                const bool paged = CHUNK && prm.chunk_paged;
                const uint16_t* v_group = paged ? cache.v_pool + paged_offset(min(group_key, SK - 1))
                                                : prm.v + kv_base + static_cast<int64_t>(group_key) * prm.kv_stride_token;
                add_non_finite_products<PRECISE>(o, __builtin_bit_cast(uint4, p.hi[kg]),
                                                 PRECISE ? __builtin_bit_cast(uint4, p.lo[kg]) : make_uint4(0, 0, 0, 0),
                                                 v_group, paged ? kDim : prm.kv_stride_token, group_key, SK, my_pos, grp);
            }
            o[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v0, p.hi[kg], o[0], 0, 0, 0);
            if (PRECISE) o[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v0, p.lo[kg], o[0], 0, 0, 0);
            o[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v1, p.hi[kg], o[1], 0, 0, 0);
            if (PRECISE) o[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v1, p.lo[kg], o[1], 0, 0, 0);
            o[2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v2, p.hi[kg], o[2], 0, 0, 0);
            if (PRECISE) o[2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v2, p.lo[kg], o[2], 0, 0, 0);
            o[3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v3, p.hi[kg], o[3], 0, 0, 0);
            if (PRECISE) o[3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v3, p.lo[kg], o[3], 0, 0, 0);
        }
    };
    // Softmax works in `units`: rounded scaled scores (ROUND) or raw fp32 dot products, whose
    // scale is folded into the exponent's multiplier (the host admits only scale > 0 there).
    const float coef = ROUND ? kLog2e : prm.scale * kLog2e;
    const float slack = ROUND ? kRescaleSlack : kRescaleSlack / prm.scale;
    // Score roundings and causal mask in place; returns the column maximum.
    auto scores = [&](f32x16_t& s, auto masked, int key_base) -> float {
        // accumulator register r of lane group grp is key key_base + 8*(r/4) + 4*grp + r%4
        const int lim = my_pos - key_base - 4 * grp;
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
    if (!CHUNK) {
        load_tile(0);
        if (prm.has_cache) fetch_pages();
        if (prm.has_cache && qt == 0) write_pages(0);
        store_tile(0);
        __syncthreads();
    }

    bool to_record = false;
    if (CHUNK) {
        // Key tiles every row of the query tile sees whole, then the one or two that the causal mask cuts
        // (two when the tile's first position is not a multiple of 64); the last tile always takes the masked
        // path, where keys beyond key_count go.  With a key split this block takes one run of them.
        const int last_tile = min(q0 + shift + BM - 1, SK - 1) / kBN;
        const int whole = PRECISE ? 0 : min((q0 + shift + 1) / kBN, last_tile);
        int t_first = 0, t_last = last_tile;
        if (!PRECISE && prm.chunk_parts > 1) {
            t_first = part * prm.chunk_run;
            if (t_first > last_tile) return;                       // (uniform over the block) no such run
            t_last = min(t_first + prm.chunk_run - 1, last_tile);
            to_record = last_tile >= prm.chunk_run;                // the query tile has more than one run
        }
        load_tile(t_first);
        store_tile(t_first & 1);
        __syncthreads();
        // (the last tile of a run takes the masked path even where no mask applies: one loop shape for every run)
        const int unmasked_end = min(whole, t_last);
        for (int t = t_first; t < unmasked_end; ++t) {
            const int stage = t & 1;
            load_tile(t + 1);
            chunk(stage, int_c<0>{}, bool_c<false>{}, 0);
            chunk(stage, int_c<1>{}, bool_c<false>{}, 0);
            store_tile(stage ^ 1);
            __syncthreads();
        }
        for (int t = max(t_first, unmasked_end);; ++t) {
            const int stage = t & 1;
            if (t < t_last) load_tile(t + 1);
            chunk(stage, int_c<0>{}, bool_c<true>{}, t * kBN);
            chunk(stage, int_c<1>{}, bool_c<true>{}, t * kBN + 32);
            if (t == t_last) break;
            store_tile(stage ^ 1);
            __syncthreads();
        }
    } else {
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
    }
    __syncthreads();   // the stages become the output staging area

    if (CHUNK && chunk_page_err && prm.status) atomicOr(prm.status, chunk_page_err);
    const float l_tot = halves_sum(l_run);
    if (CHUNK && !PRECISE && to_record) {
        // One run of several: the unnormalised O, the reference maximum and the sum, as register images (thread t of
        // the merge kernel takes what thread t leaves here).
        float* rec = prm.chunk_records
                   + ((static_cast<int64_t>(pair) * prm.n_qtiles + qt) * prm.chunk_parts + part) * kChunkRecordFloats + tid;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) rec[(16 * dt + r) * kPfThreads] = o[dt][r];
        rec[64 * kPfThreads] = m_run;
        rec[65 * kPfThreads] = l_tot;
        return;
    }

    // ---- normalise, stage through LDS, write 16 bytes per lane -------------------------------------
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
        const int row = q0 + R * wave + (c % R);
        const int head = G * kvh + c / R;
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


// The rows of a sequence continued at position cache_before (R17:17782-17813 with cache_before > 0), over keys
// and values read in place: grid and blocks as above.  A query tile none of whose rows sees a whole key tile takes
// the split-precision P path (rows with few keys).
// G query heads per kv head (1, 2 or 4): a block is 128 / G query rows.  Keys and values by strides, or (chunk_paged)
// from the paged cache `cache` through the page table.
template <bool ROUND, int G>
__global__ __launch_bounds__(kPfThreads, 2) void prefill_chunk_kernel(PrefillParams prm, qm_kv_cache cache) {
    extern __shared__ __attribute__((aligned(16))) unsigned char pf_smem[];
    const int pairs = prm.batch * prm.kv_heads;
    const int bid = blockIdx.x;
    const int group = bid / pairs;                       // heaviest query tile first, its runs side by side
    const int qt = prm.n_qtiles - 1 - group / prm.chunk_parts;
    const int part = group % prm.chunk_parts;
    const int pair = bid % pairs;
    if ((qt * (128 / G) + prm.cache_before + 1) / kBN == 0) {
        if (part == 0) prefill_body<true, ROUND, true, G>(prm, cache, pf_smem, qt, pair);
    } else {
        prefill_body<false, ROUND, true, G>(prm, cache, pf_smem, qt, pair, part);
    }
}

// Combines the runs of the query tiles that prefill_chunk_kernel split: sum over runs of O * w over sum of l * w,
// w = exp(maximum of the run - largest maximum), in run order.  grid = pairs * n_qtiles * 8, 256 threads: thread t
// holds what thread t of a run's block held (column = (row % 16, head) of a wave), and a block takes eight of the
// thread's 64 values, all runs' loads in flight at once.
constexpr int kChunkMaxRuns = 16;
constexpr int kChunkMergeSlices = 8;
__global__ __launch_bounds__(kPfThreads) void prefill_chunk_merge_kernel(PrefillParams prm, int round_scores, int gqa_group) {
    request_arguments(prm, round_scores, gqa_group);
    const int slice = blockIdx.x % kChunkMergeSlices;
    const int item = blockIdx.x / kChunkMergeSlices;
    const int pair = item % (prm.batch * prm.kv_heads);
    const int qt = item / (prm.batch * prm.kv_heads);
    const int wave_rows = 32 / gqa_group, block_rows = 4 * wave_rows;
    const int q0 = qt * block_rows;
    const int last_tile = min(q0 + prm.cache_before + block_rows - 1, prm.key_count - 1) / kBN;
    const int runs = last_tile / prm.chunk_run + 1;
    if (runs == 1) return;                               // its one block has written the rows itself
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, col = lane & 31, grp = lane >> 5;
    const float coef = round_scores ? kLog2e : prm.scale * kLog2e;
    const float* rec = prm.chunk_records + (static_cast<int64_t>(pair) * prm.n_qtiles + qt) * prm.chunk_parts * kChunkRecordFloats + tid;
    float mv[kChunkMaxRuns], lv[kChunkMaxRuns], ov[kChunkMaxRuns][8];
#pragma unroll
    for (int p = 0; p < kChunkMaxRuns; ++p) {
        const float* r = rec + static_cast<int64_t>(min(p, runs - 1)) * kChunkRecordFloats;
        mv[p] = r[64 * kPfThreads];
        lv[p] = r[65 * kPfThreads];
#pragma unroll
        for (int i = 0; i < 8; ++i) ov[p][i] = r[(8 * slice + i) * kPfThreads];
    }
    float m_all = -INFINITY;
#pragma unroll
    for (int p = 0; p < kChunkMaxRuns; ++p) m_all = fmaxf(m_all, mv[p]);
    const float m_ref = m_all == -INFINITY ? 0.0f : m_all;
    float acc[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    float l = 0.0f;
#pragma unroll
    for (int p = 0; p < kChunkMaxRuns; ++p) {
        const float w = p < runs ? fast_exp2((mv[p] - m_ref) * coef) : 0.0f;
        l = fmaf(lv[p], w, l);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = fmaf(ov[p][i], w, acc[i]);
    }
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    const int b = pair / prm.kv_heads, kvh = pair % prm.kv_heads;
    const int row = q0 + wave_rows * wave + col % wave_rows;
    if (row >= prm.seq) return;
    uint16_t* out = prm.out + ((static_cast<int64_t>(b) * prm.seq + row) * (gqa_group * prm.kv_heads) + gqa_group * kvh + col / wave_rows) * kDim;
    // value 16 dt + 4 rq + j of a thread is dim 32 dt + 8 rq + 4 grp + j: this slice is dt = slice / 2, rq = 2 (slice % 2), + 1
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        uint2 packed;
        packed.x = pack_bf16_pair(acc[4 * h + 0] * inv, acc[4 * h + 1] * inv);
        packed.y = pack_bf16_pair(acc[4 * h + 2] * inv, acc[4 * h + 3] * inv);
        *reinterpret_cast<uint2*>(out + 32 * (slice >> 1) + 8 * (2 * (slice & 1) + h) + 4 * grp) = packed;
    }
}


constexpr int kKR = kDim * 2;                                    // bytes of a K row in LDS (unpadded, slots swizzled)
constexpr int kSpKTile = kBN * kKR;                              // one 64-key tile of K (or V, row-major like K) in LDS

// s_waitcnt that waits until at most N vector-memory operations are outstanding (nothing else).
template <int N>
__device__ __forceinline__ void wait_vm() {
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// Workgroup barrier that waits for this wave's LDS traffic only: global loads issued for a later
// stage stay in flight across it (__syncthreads would drain them too).
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}


// ======================================================================================================
// The interleaved kernel: each of the four waves of a block runs the matrix and the softmax work
// of its NC column groups (16 rows x 2 heads each) as ONE software-pipelined instruction stream.
//
// Independent MFMAs and VALU instructions of the same wave do overlap when they alternate at
// fine grain (measured: 16 x (one MFMA, eight FMAs) take 684 cycles against 512 + 616 one after
// the other; an MFMA costs the wave about 11 cycles of issue), and the compiler's own order — all
// MFMAs of a product, then all of the softmax — leaves that unused.  Stage j of a wave therefore
// holds three things that do not depend on one another: the P.V MFMAs of chunk j - 1, the
// softmax arithmetic of chunk j, and the S^T MFMAs of chunk j + 1; the source alternates MFMAs
// with slices of the softmax and pins that order with scheduling fences (see the stage).
// K and V tiles go straight from global memory into LDS (global_load_lds: no registers, no
// arithmetic), V is transposed by the LDS read, with two buffers per ring and one block barrier per 64-key tile:
// 64 KiB of LDS, so that two blocks share a CU.  The block's own (diagonal) tiles are finished
// outside the pipeline, and blocks of the first query tile (split-precision P) run the
// uniform-waves body.
//
// Measured (same bits as the other kernels; batch x tokens, uniform waves / this kernel):
// 4 x 1024: 42.4 / 30.5 us, 16 x 1024: 139 / 106 us, 4 x 4096: 374 / 316 us, 1 x 8192: 366 / 305 us
// (fp32 scores: 36 / 29, 111 / 100, 339 / 291, 337 / 290).  Where the time goes, from cycle stamps
// inside the kernel: a stage (32 keys: 16 MFMAs = 512 cycles of the matrix pipe) takes 1100 cycles
// of a wave that has its SIMD to itself and 1400 on average over a tile (barrier and loads), 1500
// when two waves share the SIMD, which then completes a stage every 750 cycles (68 % of the matrix
// pipe).  The whole kernel reaches less than that for two reasons outside the pipeline: under this
// load the chip clocks at 1.65 GHz (4 x 4096) to 1.9 GHz (4 x 1024) instead of 2.4, and a block
// spends 16 000 cycles outside its pipeline (7 600 until its first loads have landed, 2 200 on
// the pages and the first S^T, 5 800 on its own tiles, the last barrier and the output), which is
// 40 % of the 4 x 1024 case, where the whole grid is resident at once and nothing hides it.
// Two column groups per wave (NC = 2: half the LDS reads per MFMA, 500 registers, one wave per
// SIMD) were slower (4 x 1024: 58 us, 4 x 4096: 389 us); the body keeps NC as a parameter, only NC = 1 is built.
constexpr int kIlRing = 2 * kSpKTile;                       // two tiles of K, likewise of V
constexpr int kIlSmemBytes = (2 * kIlRing > static_cast<int>(sizeof(PfStage)) * kPfStages)
                                 ? 2 * kIlRing : static_cast<int>(sizeof(PfStage)) * kPfStages;
static_assert(kIlSmemBytes >= 2 * 4 * 32 * kOS * 2, "the output staging area (two column groups per wave) reuses the rings");

// Key split: when the whole grid is resident at once and CUs are left over, the kernel lasts as long as the
// block of the last query tile, a serial chain over all key tiles.  A query tile of many key tiles is then given
// to up to three blocks, each taking a run of key tiles (the last one also the tile's own, diagonal keys) and
// ending with an unnormalised O, a reference maximum and a sum per column.  Blocks draw a ticket when they are
// done: all but the last to arrive publish their record and leave; the last waits for the records of blocks
// that are already running (bounded), combines  sum over parts of part * w_part  in the order of the parts (the
// same expression whoever arrives last: the result does not depend on the order of arrival) and writes the
// output.  Records go through agent-scope atomic stores and loads: they bypass the per-XCD L2s, which are not
// coherent with one another, and need no fence.
constexpr int kSplitMaxParts = 3;
constexpr int kSplitRecordFloats = 66 * kPfThreads;        // per thread: 64 of O, the reference maximum, the sum
constexpr int kSplitTicketInts = 8;                        // arrivals, one flag per part, padding
constexpr unsigned kSplitSpinLimit = 1u << 20;
__host__ __device__ inline int split_parts(int tiles, int chunk) {
    const int parts = chunk > 0 ? (tiles + chunk - 1) / chunk : 1;
    return parts > kSplitMaxParts ? kSplitMaxParts : parts;
}
// First key tile of part `part` (even: a tile's buffer is its parity); `parts` itself gives the end.  The last part
// also works through the query tile's own keys outside the pipeline and usually combines the records: it is given
// about three key tiles fewer than the others, and two at least (one for the pipeline, and the tile's own).
__host__ __device__ inline int split_first_tile(int tiles, int parts, int part) {
    const int even_share = 2 * ((part * (tiles + 3)) / (2 * parts));
    const int latest = 2 * ((tiles - 2) / 2);
    return even_share < latest ? even_share : latest;
}

// Copies the K and V rows of key tile `tile` of (batch b, kv head kvh) to their pages: 256 threads, a thread four
// rows' 16-byte pieces of either tensor.  The interleaved kernel's blocks of the lighter half of the query tiles copy
// the heavier half's key tiles with it, kHeavyTilesPerBlock each, the lightest block the last tiles.
constexpr int kHeavyTilesPerBlock = 3;
__device__ __forceinline__ void copy_tile_to_pages(const PrefillParams& prm, const qm_kv_cache& cache, int b, int kvh, int tile) {
    const int tid = threadIdx.x;
    const int32_t* table = prm.page_table ? prm.page_table + static_cast<int64_t>(b) * prm.pages.max_pages : nullptr;
    const int64_t kv_base = static_cast<int64_t>(b) * prm.kv_stride_batch + static_cast<int64_t>(kvh) * prm.kv_stride_head;
    uint32_t page_err = 0;
    // (named registers, not arrays or structures — those end up as stack objects here — and every load unconditional,
    // indices clamped into range, so that all twelve are in flight at once; phys < -1 marks a row that is not written)
    auto request = [&](int i, uint4& kx, uint4& vx, int& page, int& phys) {
        const int key = tile * kBM + (tid >> 4) + 16 * i;
        bool live = key < prm.seq;
        page = page_of(prm.pages, live ? key : 0);
        if (live && page >= prm.pages.max_pages) {
            page_err |= QM_STATUS_BAD_POSITION;
            live = false;
        }
        const int entry = live ? page : 0;
        const int found = table ? table[entry] : entry;
        phys = live ? found : -2;
        const int64_t off = kv_base + static_cast<int64_t>(min(key, prm.seq - 1)) * prm.kv_stride_token + 8 * (tid & 15);
        kx = *reinterpret_cast<const uint4*>(prm.k + off);
        vx = *reinterpret_cast<const uint4*>(prm.v + off);
    };
    auto write = [&](int i, const uint4& kx, const uint4& vx, int page, int phys) {
        if (phys == -2) return;
        if (phys < 0 || phys >= cache.n_pages) {
            page_err |= QM_STATUS_BAD_PAGE;
            return;
        }
        const int key = tile * kBM + (tid >> 4) + 16 * i;
        const int64_t off = static_cast<int64_t>(phys) * cache.stride_page + static_cast<int64_t>(kvh) * cache.stride_head
                          + static_cast<int64_t>(key - page * prm.pages.page_size) * kDim + 8 * (tid & 15);
        *reinterpret_cast<uint4*>(cache.k_pool + off) = kx;
        *reinterpret_cast<uint4*>(cache.v_pool + off) = vx;
    };
    uint4 k0, k1, k2, k3, v0, v1, v2, v3;
    int g0, g1, g2, g3, p0, p1, p2, p3;
    request(0, k0, v0, g0, p0); request(1, k1, v1, g1, p1); request(2, k2, v2, g2, p2); request(3, k3, v3, g3, p3);
    write(0, k0, v0, g0, p0); write(1, k1, v1, g1, p1); write(2, k2, v2, g2, p2); write(3, k3, v3, g3, p3);
    if (page_err && prm.status) atomicOr(prm.status, page_err);
}

template <bool ROUND, int NC>
__device__ __forceinline__ void prefill_il_body(const PrefillParams& prm, const qm_kv_cache& cache,
                                                unsigned char* il_smem, int qt, int bh,
                                                int part = 0, int parts = 1, int split_slot = 0) {
    typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
    unsigned char* lds_k = il_smem;                 // [2][64 rows][256 B]
    unsigned char* lds_v = il_smem + kIlRing;       // [2][64 rows][256 B]

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int col = lane & 31;
    const int grp = lane >> 5;

    const int b = bh / prm.kv_heads;
    const int kvh = bh % prm.kv_heads;
    const int S = prm.seq;
    const int q_heads = 2 * prm.kv_heads;
    const int q0 = qt * kBM * NC;                    // first query row of the block
    const int n_full = qt * NC;                      // key tiles wholly before the block's rows: the pipeline's
    const int last_tile = n_full + NC - 1;           // the block's own rows span the tiles n_full .. last_tile
    // the pipeline's tiles of this block: all before the block's own, or one part of them
    const bool last_part = part == parts - 1;        // the one that also takes the block's own tiles
    const int t_first = split_first_tile(n_full + 1, parts, part);
    const int t_end = last_part ? n_full : split_first_tile(n_full + 1, parts, part + 1);
    const int my_head = 2 * kvh + (col >> 4);
    // column group c of this wave: rows group_row0(c) .. + 15
    auto group_row0 = [&](int c) { return q0 + 16 * (NC * wave + c); };

    const int64_t kv_base = static_cast<int64_t>(b) * prm.kv_stride_batch + static_cast<int64_t>(kvh) * prm.kv_stride_head;
    const int kv_row32 = static_cast<int>(prm.kv_stride_token);

    // ---- K/V rows for the pages.  Writing key tile t to the pages is exact and independent of everything else, so
    // it need not be done by the block of query tile t.
    // When the whole grid is resident at once (dealt_pages) the kernel lasts as long as the blocks of the heaviest
    // query tiles, and those write none: every block of the lighter half writes its own tile, and the heavy tiles
    // are dealt three at a time to the lightest blocks (which have the most time to spare), before anything else
    // of theirs: their requests join the burst of first requests of the whole grid, and they wait for them while
    // the heavy blocks already run.
    // Otherwise blocks queue for the CUs, a block that waits is a CU slot that idles, and every block writes its
    // own tile: rows requested behind its first tiles, written after its first wait. ----
    static_assert(NC == 1, "the page write takes key tiles of 64 rows");
    const int light_tiles = prm.n_qtiles - prm.n_qtiles / 2;
    if (prm.has_cache != 0 && prm.dealt_pages != 0 && last_part && qt < light_tiles) {
        copy_tile_to_pages(prm, cache, b, kvh, qt);
#pragma unroll 1
        for (int j = 0; j < kHeavyTilesPerBlock; ++j) {
            const int heavy = prm.n_qtiles - 1 - (kHeavyTilesPerBlock * qt + j);
            if (heavy >= light_tiles) copy_tile_to_pages(prm, cache, b, kvh, heavy);
        }
    }
    const bool own_pages = prm.has_cache != 0 && prm.dealt_pages == 0 && last_part;
    int phys[4];
    uint4 kx[4], vx[4];
    uint32_t page_err = 0;
    auto request_page_rows = [&]() {
        const int32_t* table = prm.page_table ? prm.page_table + static_cast<int64_t>(b) * prm.pages.max_pages : nullptr;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int key = q0 + (tid >> 4) + 16 * i;
            phys[i] = -1;
            kx[i] = vx[i] = make_uint4(0, 0, 0, 0);
            if (key < S) {
                const int page = page_of(prm.pages, key);
                if (page >= prm.pages.max_pages) page_err |= QM_STATUS_BAD_POSITION;
                else phys[i] = table ? table[page] : page;
                const int64_t off = kv_base + static_cast<int64_t>(key) * prm.kv_stride_token + 8 * (tid & 15);
                kx[i] = *reinterpret_cast<const uint4*>(prm.k + off);
                vx[i] = *reinterpret_cast<const uint4*>(prm.v + off);
            }
        }
    };
    auto write_page_rows = [&]() {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int key = q0 + (tid >> 4) + 16 * i;
            if (key >= S || phys[i] == -1) continue;
            if (phys[i] < 0 || phys[i] >= cache.n_pages) {
                page_err |= QM_STATUS_BAD_PAGE;
                continue;
            }
            const int page = page_of(prm.pages, key);
            const int64_t off = static_cast<int64_t>(phys[i]) * cache.stride_page + static_cast<int64_t>(kvh) * cache.stride_head
                              + static_cast<int64_t>(key - page * prm.pages.page_size) * kDim + 8 * (tid & 15);
            *reinterpret_cast<uint4*>(cache.k_pool + off) = kx[i];
            *reinterpret_cast<uint4*>(cache.v_pool + off) = vx[i];
        }
        if (page_err && prm.status) atomicOr(prm.status, page_err);
    };

    // ---- staging: one global_load_lds of a wave (16 bytes per lane) fills four consecutive 256-byte rows of a
    // tile, lane l row l / 16, slot l % 16; which 16-byte piece of the key the lane fetches into that slot is
    // the swizzle.  Slot p of K row r holds piece p ^ (r % 16), so that the fragment reads of 16 consecutive
    // rows fall on 16 different slots; V stays row-major too (slot p of row r holds piece p ^ 4 (r % 4)) and is
    // transposed by the LDS read.  A key at or beyond S is redirected to the last key; such keys only occur
    // masked.  Wave w fills rows 4 w + l / 16 + 16 j of a tile ----
    const int k_row = 4 * wave + (lane >> 4);
    const uint32_t row_bytes = static_cast<uint32_t>(kv_row32) * 2u;
    // Requests go through buffer descriptors that cover exactly the S keys of this (batch, kv head): a lane's offset
    // is the piece's first key (the instruction's scalar offset) plus a 32-bit value that never changes (its row inside
    // the piece and the 16-byte piece of the key it fetches: the vector offset), and a key at or beyond S is out
    // of the descriptor's range: it reads as zero and touches no memory (such keys only occur masked).
    const uint32_t kv_bytes = static_cast<uint32_t>(S - 1) * row_bytes + static_cast<uint32_t>(kKR);
    const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(prm.k + kv_base), 0, static_cast<int>(kv_bytes), 0x00020000);
    const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(prm.v + kv_base), 0, static_cast<int>(kv_bytes), 0x00020000);
    const uint32_t k_lane = static_cast<uint32_t>(k_row) * row_bytes + 16u * ((lane & 15) ^ (k_row & 15));
    const uint32_t v_lane = static_cast<uint32_t>(k_row) * row_bytes + 16u * ((lane & 15) ^ (4 * (k_row & 3)));
    // piece j of a tile: one request of a wave (16 bytes per lane, no registers) fills rows 4 w + 16 j .. + 3
    // (`wanted` false: the request stays in the instruction stream, which a branch around it would cut in two, and
    // asks for the bytes that follow the descriptor's range: zeros into a buffer nobody reads, no memory touched)
    auto load_piece = [&](const __amdgpu_buffer_rsrc_t& rsrc, uint32_t lane_off, unsigned char* ring, int tile, int slot, int j,
                          bool wanted = true) {
        unsigned char* dst = ring + slot * kSpKTile + (4 * wave + 16 * j) * kKR;
        const uint32_t piece = wanted ? static_cast<uint32_t>(tile * kBN + 16 * j) * row_bytes : kv_bytes;
        // (the piece's offset travels as the instruction's scalar offset, which takes part in the range check like the
        // vector offset: no vector addition)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)dst, 16,
                                                 static_cast<int>(lane_off), static_cast<int>(piece), 0, 0);
    };
    auto load_k_piece = [&](int tile, int slot, int j, bool wanted = true) { load_piece(k_rsrc, k_lane, lds_k, tile, slot, j, wanted); };
    auto load_v_piece = [&](int tile, int slot, int j) { load_piece(v_rsrc, v_lane, lds_v, tile, slot, j); };
    auto load_k = [&](int tile, int slot) {
#pragma unroll
        for (int j = 0; j < 4; ++j) load_k_piece(tile, slot, j);
    };
    auto load_v = [&](int tile, int slot) {
#pragma unroll
        for (int j = 0; j < 4; ++j) load_v_piece(tile, slot, j);
    };

    // What the first product needs is requested first: K of the first tile and the wave's own Q fragments.  A block
    // that has no page rows to wait for waits for those alone (loads come back in the order of their requests) and
    // leaves V of the first tile and K of the second in flight: the first tile's barrier inside the pipeline waits
    // for them.
    load_k(t_first, 0);                              // t_first is even: tile t lives in buffer t % 2
    bf16x8_t qf[NC][8];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int row = group_row0(c) + (col & 15);
        const uint16_t* qp = prm.q + ((static_cast<int64_t>(b) * S + row) * q_heads + my_head) * kDim + 8 * grp;
#pragma unroll
        for (int kb = 0; kb < 8; ++kb) {
            uint4 raw = make_uint4(0, 0, 0, 0);
            if (row < S) raw = *reinterpret_cast<const uint4*>(qp + 16 * kb);
            qf[c][kb] = __builtin_bit_cast(bf16x8_t, raw);
        }
    }
    load_v(t_first, 0);
    load_k(t_first + 1, 1);                          // qt >= 1, and every part holds two tiles at least: it exists
    f32x16_t o[NC][4];
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[c][dt][r] = 0.0f;
    if (own_pages) {
        request_page_rows();
        wait_vm<0>();
        write_page_rows();
    } else {
        // (a row at or beyond S requests no Q: then fewer loads are outstanding than the count assumes and the
        // wait is merely longer)
        wait_vm<8>();
    }
    lds_barrier();

    // ---- fragment reads, all as assembly: the compiler would make an LDS read wait for every
    // global_load_lds in flight, and it must not move them across the barriers either.  Their results
    // are taken only through the *_arrived statements, which wait for them. ----
    // K fragment kb of chunk (slot, h): row 32 h + col, slot (2 kb + grp) ^ (col % 16).
    // V^T fragment (kg, dt): one ds_read_b64_tr_b16 of 16 lanes takes a block of 4 keys x 16 dims (lane 4 j + q of
    // the 16 addresses dims 4 q .. 4 q + 3 of key j) and gives lane i the four keys of dim i.  MFMA k index
    // 8 grp + e of 16-key group kg is key 16 kg + 8 (e / 4) + 4 grp + e % 4 (the S^T accumulator's order), so the
    // fragment of lane (dim col, grp) is two such reads, keys 16 kg + 4 grp + 0..3 and + 8.
    uint32_t kaddr[8], vaddr[4];
    {
        const uint32_t k0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) unsigned char*)lds_k))
                          + col * kKR + 16 * (grp ^ (col & 15));
#pragma unroll
        for (int kb = 0; kb < 8; ++kb) kaddr[kb] = k0 ^ (32 * kb);
        const int tr_key = (lane >> 2) & 3;
        const uint32_t v0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) unsigned char*)lds_v))
                          + (4 * grp + tr_key) * kKR + 16 * (2 * (col >> 4) + ((lane & 3) >> 1)) + 8 * (lane & 1);
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) vaddr[dt] = v0 ^ (64 * (dt ^ tr_key));
    }
    struct KRaw { u32x4_t f[8]; };
    struct VRaw { unsigned long long a[8], c[8]; };
    // One K fragment (k block i) / one V^T fragment (i = 4 kg + dt: two reads).  `dyn`: bytes added at run
    // time (0 in the pipeline, where the buffer is a template constant).
    auto k_request_one = [&](uint32_t dyn, auto imm, int i, KRaw& raw) {
        const uint32_t at = kaddr[i] + dyn;
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(raw.f[i]) : "v"(at), "n"(decltype(imm)::value));
    };
    auto v_request_one = [&](uint32_t dyn, auto imm, int i, VRaw& raw) {
        const uint32_t at = vaddr[i & 3] + dyn;
        if (i < 4) {
            asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(raw.a[i]) : "v"(at), "n"(decltype(imm)::value));
            asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(raw.c[i]) : "v"(at), "n"(decltype(imm)::value + 8 * kKR));
        } else {
            asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(raw.a[i]) : "v"(at), "n"(decltype(imm)::value + 16 * kKR));
            asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(raw.c[i]) : "v"(at), "n"(decltype(imm)::value + 24 * kKR));
        }
    };
    auto k_request = [&](uint32_t dyn, auto imm, KRaw& raw) {
#pragma unroll
        for (int i = 0; i < 8; ++i) k_request_one(dyn, imm, i, raw);
    };
    auto v_request = [&](uint32_t dyn, auto imm, VRaw& raw) {
#pragma unroll
        for (int i = 0; i < 8; ++i) v_request_one(dyn, imm, i, raw);
    };
    auto v_unpack = [&](const VRaw& raw, int j) -> bf16x8_t {
        const uint4 both_halves = make_uint4(static_cast<uint32_t>(raw.a[j]), static_cast<uint32_t>(raw.a[j] >> 32),
                                             static_cast<uint32_t>(raw.c[j]), static_cast<uint32_t>(raw.c[j] >> 32));
        return __builtin_bit_cast(bf16x8_t, both_halves);
    };
    // Waits until at most `pending` LDS reads are outstanding, then hands out half h of both sets.
    auto half_arrived = [&](auto half, auto pending, KRaw& kraw, VRaw& vraw, bf16x8_t (&kf)[8], bf16x8_t (&vf)[8]) {
        constexpr int h = 4 * decltype(half)::value;
        asm volatile("s_waitcnt lgkmcnt(%12)"
                     : "+v"(kraw.f[h]), "+v"(kraw.f[h + 1]), "+v"(kraw.f[h + 2]), "+v"(kraw.f[h + 3]),
                       "+v"(vraw.a[h]), "+v"(vraw.a[h + 1]), "+v"(vraw.a[h + 2]), "+v"(vraw.a[h + 3]),
                       "+v"(vraw.c[h]), "+v"(vraw.c[h + 1]), "+v"(vraw.c[h + 2]), "+v"(vraw.c[h + 3])
                     : "n"(decltype(pending)::value)
                     : "memory");
#pragma unroll
        for (int i = h; i < h + 4; ++i) {
            kf[i] = __builtin_bit_cast(bf16x8_t, kraw.f[i]);
            vf[i] = v_unpack(vraw, i);
        }
    };
    auto k_arrived = [&](KRaw& raw, bf16x8_t (&kf)[8]) {
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(raw.f[0]), "+v"(raw.f[1]), "+v"(raw.f[2]), "+v"(raw.f[3]), "+v"(raw.f[4]), "+v"(raw.f[5]),
                       "+v"(raw.f[6]), "+v"(raw.f[7])
                     :
                     : "memory");
#pragma unroll
        for (int kb = 0; kb < 8; ++kb) kf[kb] = __builtin_bit_cast(bf16x8_t, raw.f[kb]);
    };
    auto v_arrived = [&](VRaw& raw, bf16x8_t (&vf)[8]) {
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(raw.a[0]), "+v"(raw.a[1]), "+v"(raw.a[2]), "+v"(raw.a[3]), "+v"(raw.a[4]), "+v"(raw.a[5]),
                       "+v"(raw.a[6]), "+v"(raw.a[7]), "+v"(raw.c[0]), "+v"(raw.c[1]), "+v"(raw.c[2]), "+v"(raw.c[3]),
                       "+v"(raw.c[4]), "+v"(raw.c[5]), "+v"(raw.c[6]), "+v"(raw.c[7])
                     :
                     : "memory");
#pragma unroll
        for (int j = 0; j < 8; ++j) vf[j] = v_unpack(raw, j);
    };

    // ---- softmax state (per column group) and the arithmetic of the uniform waves, cut into score pairs ----
    const float coef = ROUND ? kLog2e : prm.scale * kLog2e;
    const float slack = ROUND ? kRescaleSlack : kRescaleSlack / prm.scale;
    // (m_limit: what a stage's maximum must exceed for the running maximum to be raised, m_run + slack; kept by the
    // pipeline's stages only, which are the first to change m_run)
    float m_run[NC], l_run[NC], m_scaled_neg[NC], m_limit[NC];   // (m_scaled_neg: minus the reference maximum times the exponent's factor)
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        m_run[c] = -INFINITY;
        l_run[c] = 0.0f;
        m_scaled_neg[c] = 0.0f;
        m_limit[c] = -INFINITY;
    }
    // roundings and the causal mask of the score pair r, r + 1 in place (the diagonal tiles)
    auto score_pair_masked = [&](f32x16_t& s, int r, float& mx, int lim) {
        float x0 = s[r], x1 = s[r + 1];
        if (ROUND) {
            round_bf16_pair(x0, x1, x0, x1);
            round_bf16_pair(x0 * prm.scale, x1 * prm.scale, x0, x1);
        }
        const int e = 8 * (r >> 2) + (r & 3);
        if (e > lim) x0 = -INFINITY;
        if (e + 1 > lim) x1 = -INFINITY;
        s[r] = x0;
        s[r + 1] = x1;
        mx = fmaxf(mx, fmaxf(x0, x1));
    };
    // raises the running maximum of column group c if some column exceeds it by more than the slack, and
    // rescales O and the running sum for it (the diagonal tiles; the pipeline defers the rescaling of O)
    auto update_max = [&](int c, float mx) {
        const bool need = __builtin_amdgcn_ballot_w64(mx > m_run[c] + slack) != 0;
        if (need) {
            const float m_new = fmaxf(m_run[c], mx);
            const float m_ref = m_new == -INFINITY ? 0.0f : m_new;
            const float alpha = fast_exp2((m_run[c] - m_ref) * coef);
            m_run[c] = m_new;
            m_scaled_neg[c] = -(m_ref * coef);
            l_run[c] *= alpha;
#pragma unroll
            for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) o[c][dt][r] *= alpha;
        }
    };
    auto prob_pair = [&](int c, const f32x16_t& s, int r, uint32_t& packed, float& psum) {
        const float e0 = fast_exp2(fmaf(s[r], coef, m_scaled_neg[c]));
        const float e1 = fast_exp2(fmaf(s[r + 1], coef, m_scaled_neg[c]));
        packed = pack_bf16_pair(e0, e1);
        psum = dot2_bf16(packed, 0x3f803f80U, psum);          // the sum of what the MFMA multiplies
    };
    struct PPair { bf16x8_t g[2]; };
    auto make_p = [&](const uint32_t (&hi)[8], PPair& p) {
        p.g[0] = __builtin_bit_cast(bf16x8_t, make_uint4(hi[0], hi[1], hi[2], hi[3]));
        p.g[1] = __builtin_bit_cast(bf16x8_t, make_uint4(hi[4], hi[5], hi[6], hi[7]));
    };

    // ---- one stage of the pipeline ----
    // in:  s_cur = raw S^T of chunk j; p_prev = P of chunk j - 1; vraw = V^T fragments of chunk j - 1 and
    //      kraw = K fragments of chunk j + 1, both requested (first halves a half stage before the second)
    // out: s_next = raw S^T of chunk j + 1; p_cur = P of chunk j; vraw = V^T fragments of chunk j (from `v_imm`)
    //      and kraw = K fragments of chunk j + 2 (from `k_imm`), requested
    // What the order of the instructions answers to (all measured on this chip):
    //  - a fragment read from LDS feeds the MFMAs of all NC column groups of the wave: with one group (32
    //    columns) every MFMA needs 1 KiB of LDS, the four SIMDs of a CU together 128 bytes per cycle, which is
    //    all its LDS delivers; with two groups it is half of that;
    //  - dependent VALU instructions issue 8 cycles apart, independent ones 4 (the exponential takes 12), and
    //    the arithmetic of one score pair is a single chain six instructions deep: the stage works on two
    //    pairs at a time, level by level, so that an independent instruction sits between dependent ones;
    //  - a dependent MFMA waits for the one before it to finish: the S^T MFMAs (one accumulator per column
    //    group) alternate with the P.V MFMAs (four accumulators), one MFMA per half group of VALU work;
    //  - eight global_load_lds in a row take 500 cycles to issue and twelve LDS reads in a row 200: the loads
    //    of a tile are handed out one per group (`vmem`), a fragment is requested as soon as the last MFMA
    //    that uses its registers has been issued, and the block barrier of the tile (`sync`) comes after
    //    the first group, when the LDS reads it has to wait for have long landed;
    //  - the chain from the maxima to the branch on them is 14 dependent instructions: MFMAs are issued
    //    ahead of it.  If the running maximum is raised, O is rescaled at the end of the stage, after the last
    //    P.V MFMA of chunk j - 1 (whose P is relative to the old maximum).
    // Scheduling fences pin the order.
    auto fence = []() { __builtin_amdgcn_sched_barrier(0); };
    auto stage = [&](f32x16_t (&s_cur)[NC], f32x16_t (&s_next)[NC], const PPair (&p_prev)[NC], PPair (&p_cur)[NC],
                     KRaw& kraw, VRaw& vraw, auto k_imm, auto v_imm, auto&& sync, auto&& vmem) {
        bf16x8_t kf[8], vf[8];
        auto pv_mfma = [&](int i, int c) {
            o[c][i & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[i], p_prev[c].g[i >> 2], o[c][i & 3], 0, 0, 0);
        };
        auto qk_mfma = [&](int i, int c) {
            // (the first product of a chunk starts from a literal zero instead of sixteen zeroed registers)
            const f32x16_t zero = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
            s_next[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[i], qf[c][i], i == 0 ? zero : s_next[c], 0, 0, 0);
        };
        half_arrived(int_c<0>{}, int_c<12>{}, kraw, vraw, kf, vf);
        // (ROUND) the maxima of the raw scores are taken in the first group and then walk, one step per group,
        // through the roundings (monotonic: the result is the maximum of the rounded scores; the host sends a
        // negative scale elsewhere) and the exchange between the two halves of the wave, so that the branch
        // on them after the last group waits for nothing
        float mx_a[NC], mx_b[NC], mx_step[NC];
        uint32_t hi[NC][8];
        float psum[NC];
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            mx_a[c] = mx_b[c] = -INFINITY;
            mx_step[c] = 0.0f;
            psum[c] = 0.0f;
        }
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int ra = 4 * g, rb = 4 * g + 2;              // pair a = scores ra, ra + 1; pair b = rb, rb + 1
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                pv_mfma(g, c);
                fence();
                if (ROUND) {
                    // (a rounding is one instruction per score: v_cvt_pk_bf16_f32 of (0, x) leaves bf16(x) in the
                    // upper half of the register, which is the rounded value as fp32; rounding two scores into
                    // one register costs the conversion and two instructions to take them apart again)
                    const float xa0 = s_cur[c][ra], xa1 = s_cur[c][ra + 1], xb0 = s_cur[c][rb], xb1 = s_cur[c][rb + 1];
                    float ua0 = round_bf16_single(xa0);
                    const float ua1 = round_bf16_single(xa1), ub0 = round_bf16_single(xb0), ub1 = round_bf16_single(xb1);
                    if (g == 0) {
                        // (assembly: the compiler's fmaxf first quiets every operand with an instruction of its
                        // own.  `ua0` passes through the first statement so that the chain follows a read of the
                        // MFMA results that the compiler guards; one MFMA wrote all sixteen.)
                        asm volatile("v_max_f32 %0, %2, %3" : "=v"(mx_a[c]), "+v"(ua0) : "v"(s_cur[c][0]), "v"(s_cur[c][1]));
                        asm volatile("v_max_f32 %0, %1, %2" : "=v"(mx_b[c]) : "v"(s_cur[c][2]), "v"(s_cur[c][3]));
#pragma unroll
                        for (int r = 4; r < 16; r += 4) {
                            asm volatile("v_max3_f32 %0, %0, %1, %2" : "+v"(mx_a[c]) : "v"(s_cur[c][r]), "v"(s_cur[c][r + 1]));
                            asm volatile("v_max3_f32 %0, %0, %1, %2" : "+v"(mx_b[c]) : "v"(s_cur[c][r + 2]), "v"(s_cur[c][r + 3]));
                        }
                    }
                    if (g == 1) {
                        asm volatile("v_max_f32 %0, %1, %2" : "=v"(mx_step[c]) : "v"(mx_a[c]), "v"(mx_b[c]));
                    }
                    if (g == 3) {
                        mx_step[c] = round_bf16_single(mx_step[c]);
                        asm volatile("" : "+v"(mx_step[c]));
                    }
                    fence();
                    const float ya0 = ua0 * prm.scale, ya1 = ua1 * prm.scale;
                    fence();
                    qk_mfma(g, c);
                    fence();
                    const float yb0 = ub0 * prm.scale, yb1 = ub1 * prm.scale;
                    if (g == 1) {
                        mx_step[c] = round_bf16_single(mx_step[c]);
                        asm volatile("" : "+v"(mx_step[c]));
                    }
                    if (g == 2) {
                        mx_step[c] = mx_step[c] * prm.scale;
                        asm volatile("" : "+v"(mx_step[c]));
                    }
                    fence();
                    float za0 = round_bf16_single(ya0), za1 = round_bf16_single(ya1);
                    float zb0 = round_bf16_single(yb0), zb1 = round_bf16_single(yb1);
                    // (an empty statement that keeps the roundings here instead of sinking to where they are used)
                    asm volatile("" : "+v"(za0), "+v"(za1), "+v"(zb0), "+v"(zb1));
                    if (g == 3) {
                        const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx_step[c]), __float_as_uint(mx_step[c]), false, false);
                        asm volatile("v_max_f32 %0, %1, %2" : "=v"(mx_step[c]) : "v"(__uint_as_float(sw[0])), "v"(__uint_as_float(sw[1])));
                    }
                    s_cur[c][ra] = za0; s_cur[c][ra + 1] = za1; s_cur[c][rb] = zb0; s_cur[c][rb + 1] = zb1;
                } else {
                    // (assembly for the same reason as above.  The first maximum starts from a score through a
                    // statement the compiler sees, so that it guards the read of the MFMA's results.)
                    if (g == 0) {
                        mx_a[c] = s_cur[c][0];
                        asm volatile("v_max3_f32 %0, %0, %1, %2" : "+v"(mx_a[c]) : "v"(s_cur[c][1]), "v"(s_cur[c][1]));
                    } else {
                        asm volatile("v_max3_f32 %0, %0, %1, %2" : "+v"(mx_a[c]) : "v"(s_cur[c][ra]), "v"(s_cur[c][ra + 1]));
                    }
                    fence();
                    qk_mfma(g, c);
                    fence();
                    asm volatile("v_max3_f32 %0, %0, %1, %2" : "+v"(mx_b[c]) : "v"(s_cur[c][rb]), "v"(s_cur[c][rb + 1]));
                }
                fence();
            }
            if (g == 0) sync();
            vmem(g);
            k_request_one(0u, k_imm, g, kraw);
            v_request_one(0u, v_imm, g, vraw);
            fence();
        }
        half_arrived(int_c<1>{}, int_c<12>{}, kraw, vraw, kf, vf);
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            qk_mfma(4, c);
            pv_mfma(4, c);
        }
        fence();

        // (a raised maximum: the new reference is needed at once, for the probabilities; the factor that O and the
        // running sum shrink by is formed where it is used, at the end of the stage, from the exponent kept here)
        bool need[NC];
        float shrink[NC];
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            float mx = mx_step[c];
            if (!ROUND) {
                asm volatile("v_max_f32 %0, %1, %2" : "=v"(mx) : "v"(mx_a[c]), "v"(mx_b[c]));
                const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(mx), __float_as_uint(mx), false, false);
                asm volatile("v_max_f32 %0, %1, %2" : "=v"(mx) : "v"(__uint_as_float(sw[0])), "v"(__uint_as_float(sw[1])));
            }
            need[c] = __builtin_amdgcn_ballot_w64(mx > m_limit[c]) != 0;
            asm volatile("" : "=v"(shrink[c]));        // (read only where need[c]: a register, no instruction)
            if (need[c]) {
                const float m_new = fmaxf(m_run[c], mx);
                const float m_ref = m_new == -INFINITY ? 0.0f : m_new;
                shrink[c] = (m_run[c] - m_ref) * coef;
                m_run[c] = m_new;
                m_limit[c] = m_new + slack;
                m_scaled_neg[c] = -(m_ref * coef);
            }
        }
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int ra = 4 * g, rb = 4 * g + 2;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                if (g > 0) pv_mfma(4 + g, c);
                fence();
                const float ta0 = fmaf(s_cur[c][ra], coef, m_scaled_neg[c]), ta1 = fmaf(s_cur[c][ra + 1], coef, m_scaled_neg[c]);
                const float tb0 = fmaf(s_cur[c][rb], coef, m_scaled_neg[c]), tb1 = fmaf(s_cur[c][rb + 1], coef, m_scaled_neg[c]);
                fence();
                const float ea0 = fast_exp2(ta0), ea1 = fast_exp2(ta1);
                fence();
                if (g < 3) qk_mfma(5 + g, c);
                fence();
                const float eb0 = fast_exp2(tb0), eb1 = fast_exp2(tb1);
                fence();
                hi[c][2 * g] = pack_bf16_pair(ea0, ea1);
                hi[c][2 * g + 1] = pack_bf16_pair(eb0, eb1);
                fence();
                psum[c] = dot2_bf16(hi[c][2 * g], 0x3f803f80U, psum[c]);          // the sum of what the MFMA multiplies
                psum[c] = dot2_bf16(hi[c][2 * g + 1], 0x3f803f80U, psum[c]);
                // (an empty statement that keeps this arithmetic here: its results are only used by the next
                // stage, and the compiler would sink it below the branch at the end of this one)
                asm volatile("" : "+v"(hi[c][2 * g]), "+v"(hi[c][2 * g + 1]), "+v"(psum[c]));
                fence();
            }
            vmem(4 + g);
            k_request_one(0u, k_imm, 4 + g, kraw);
            v_request_one(0u, v_imm, 4 + g, vraw);
            fence();
        }
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            make_p(hi[c], p_cur[c]);
            if (need[c]) {
                const float alpha = fast_exp2(shrink[c]);
                l_run[c] *= alpha;
#pragma unroll
                for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) o[c][dt][r] *= alpha;
            }
            l_run[c] += psum[c];
        }
    };

    // ---- prologue: S^T of chunk (0, 0); K fragments of chunk (0, 1) requested; nothing to multiply yet ----
    f32x16_t s_a[NC], s_b[NC];
    PPair p_a[NC], p_b[NC];
    KRaw kraw;
    VRaw vraw;
    {
        bf16x8_t kf[8];
        k_request(0u, int_c<0>{}, kraw);
        k_arrived(kraw, kf);
#pragma unroll
        for (int c = 0; c < NC; ++c) {
#pragma unroll
            for (int r = 0; r < 16; ++r) s_a[c][r] = 0.0f;
#pragma unroll
            for (int kb = 0; kb < 8; ++kb) s_a[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[kb], qf[c][kb], s_a[c], 0, 0, 0);
            p_b[c].g[0] = p_b[c].g[1] = __builtin_bit_cast(bf16x8_t, make_uint4(0, 0, 0, 0));
        }
        k_request(0u, int_c<32 * kKR>{}, kraw);
        // (the stages count outstanding reads in halves of twelve; these eight are taken here)
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(kraw.f[0]), "+v"(kraw.f[1]), "+v"(kraw.f[2]), "+v"(kraw.f[3]), "+v"(kraw.f[4]), "+v"(kraw.f[5]),
                       "+v"(kraw.f[6]), "+v"(kraw.f[7])
                     :
                     : "memory");
#pragma unroll
        for (int j = 0; j < 8; ++j) vraw.a[j] = vraw.c[j] = 0ull;
    }

    // ---- the tiles before the block's own: tile t lives in buffer t % 2 of either ring.  During its first stage
    // (after the tile's barrier: every wave has taken the last fragments of tile t - 1 and of K tile t) the
    // wave requests K of tile t + 2 into the buffer of K tile t and V of tile t + 1 into the buffer of V tile
    // t - 1; both are first read during tile t + 1, after its barrier. ----
    auto tile_body = [&](int t, auto parity) {
        constexpr int cur = decltype(parity)::value;
        constexpr int nxt = cur ^ 1;
        const bool more_k = t + 2 <= last_tile;
        // stage (t, 0): P.V of chunk (t - 1, 1), softmax of (t, 0), S^T of (t, 1); requests V(t, 0) and K(t + 1, 0)
        stage(s_a, s_b, p_b, p_a, kraw, vraw, int_c<nxt * kSpKTile>{}, int_c<cur * kSpKTile>{},
              [&]() {
                  wait_vm<0>();
                  lds_barrier();
              },
              [&](int i) {
                  if (i < 4) {
                      load_k_piece(t + 2, cur, i, more_k);
                  } else {
                      load_v_piece(t + 1, nxt, i - 4);
                  }
              });
        // stage (t, 1): P.V of chunk (t, 0), softmax of (t, 1), S^T of (t + 1, 0); requests V(t, 1) and K(t + 1, 1)
        stage(s_b, s_a, p_a, p_b, kraw, vraw, int_c<nxt * kSpKTile + 32 * kKR>{}, int_c<cur * kSpKTile + 32 * kKR>{},
              []() {}, [](int) {});
    };
    // (a part before the last requests, and multiplies into scores nobody reads, up to two tiles past its end: they exist)
    for (int t = t_first; t < t_end; t += 2) {
        tile_body(t, int_c<0>{});
        if (t + 1 < t_end) tile_body(t + 1, int_c<1>{});
    }
    wait_vm<0>();
    lds_barrier();                                   // what has been loaded has landed for every wave, and every
                                                     // wave has taken its fragments of V tile n_full - 1
    if (NC == 2) load_v(last_tile, last_tile & 1);   // (the pipeline requested V up to tile n_full only)

    // ---- drain: P.V of chunk (t_end - 1, 1), then the block's own tiles chunk by chunk ----
    {
        bf16x8_t vf[8];
        v_arrived(vraw, vf);
#pragma unroll
        for (int c = 0; c < NC; ++c)
#pragma unroll
            for (int i = 0; i < 8; ++i)
                o[c][i & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[i], p_b[c].g[i >> 2], o[c][i & 3], 0, 0, 0);
    }
    // Chunk d of the block's own tiles (first key key_base) concerns column group c if key_base is not after the
    // group's last row; it is masked for that group.  A 16-key group wholly after the last row is masked for every
    // column: skipped, so that later tokens are not even multiplied by zero.
    auto diag_group = [&](int c, f32x16_t& s, const bf16x8_t (&vf)[8], int key_base) {
        const int lim = group_row0(c) + (col & 15) - key_base - 4 * grp;
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 8; ++i) score_pair_masked(s, 2 * i, mx, lim);
        mx = halves_max(mx);
        update_max(c, mx);
        uint32_t hi[8];
        float psum = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) prob_pair(c, s, 2 * i, hi[i], psum);
        l_run[c] += psum;
        PPair p;
        make_p(hi, p);
#pragma unroll
        for (int kg = 0; kg < 2; ++kg) {
            if (key_base + 16 * kg > group_row0(c) + 15) continue;
            // (the group the mask cuts — the one of the wave's own rows, or one that reaches beyond S — with a
            // non-finite V: see add_non_finite_products)
            bf16x8_t v0 = vf[4 * kg], v1 = vf[4 * kg + 1], v2 = vf[4 * kg + 2], v3 = vf[4 * kg + 3];
            if ((key_base + 16 * kg + 15 > group_row0(c) || key_base + 16 * kg + 15 >= S) && any_non_finite(v0, v1, v2, v3)) {
                zero_non_finite(v0); zero_non_finite(v1); zero_non_finite(v2); zero_non_finite(v3);
                add_non_finite_products<false>(o[c], __builtin_bit_cast(uint4, p.g[kg]), make_uint4(0, 0, 0, 0),
                                               prm.v + kv_base + static_cast<int64_t>(key_base + 16 * kg) * prm.kv_stride_token,
                                               prm.kv_stride_token, key_base + 16 * kg, S, group_row0(c) + (col & 15), grp);
            }
            o[c][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v0, p.g[kg], o[c][0], 0, 0, 0);
            o[c][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v1, p.g[kg], o[c][1], 0, 0, 0);
            o[c][2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v2, p.g[kg], o[c][2], 0, 0, 0);
            o[c][3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v3, p.g[kg], o[c][3], 0, 0, 0);
        }
    };
    if (last_part)
#pragma unroll
    for (int d = 0; d < 2 * NC; ++d) {
        const int tile = n_full + (d >> 1);
        const int key_base = tile * kBN + 32 * (d & 1);
        const uint32_t slot_bytes = static_cast<uint32_t>((tile & 1) * kSpKTile);
        if (d == 2) {
            wait_vm<0>();
            lds_barrier();                           // V of the last tile has landed for every wave
        }
        const bool any = key_base <= group_row0(NC - 1) + 15;       // (the wave's last column group sees the most)
        bf16x8_t kf[8], vf[8];
        if (d >= 1) {
            // K fragments: those of chunk 1 were requested by the pipeline (every wave takes them, so that no
            // read is left pending); later ones are requested here
            if (d >= 2 && any) {
                if (d & 1) k_request(slot_bytes, int_c<32 * kKR>{}, kraw);
                else k_request(slot_bytes, int_c<0>{}, kraw);
            }
            if (d == 1 || any) k_arrived(kraw, kf);
        }
        if (!any) continue;
        VRaw vr;
        if (d & 1) v_request(slot_bytes, int_c<32 * kKR>{}, vr);
        else v_request(slot_bytes, int_c<0>{}, vr);
        if (d >= 1) {
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                if (key_base > group_row0(c) + 15) continue;
#pragma unroll
                for (int r = 0; r < 16; ++r) s_a[c][r] = 0.0f;
#pragma unroll
                for (int kb = 0; kb < 8; ++kb) s_a[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[kb], qf[c][kb], s_a[c], 0, 0, 0);
            }
        }
        v_arrived(vr, vf);
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            if (key_base > group_row0(c) + 15) continue;
            diag_group(c, s_a[c], vf, key_base);
        }
    }
    // ---- a split query tile: all blocks but the last to arrive publish, the last combines ----
    if (NC == 1 && parts > 1) {
        lds_barrier();   // every wave is done with the rings: their first words carry the notes below
        const int64_t slot = static_cast<int64_t>(bh) * prm.split_slots + split_slot;
        float* records = prm.split_partials + slot * kSplitMaxParts * kSplitRecordFloats + tid;
        int* tickets = prm.split_tickets + slot * kSplitTicketInts;
        int* note = reinterpret_cast<int*>(il_smem);
        if (tid == 0) {
            // The ticket word is (epoch << 4) | arrivals of this launch: a word left by another launch (or by one
            // that gave up waiting) counts as no arrivals, so nothing has to be reset and nothing stale is believed.
            int seen = __hip_atomic_load(&tickets[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            for (;;) {
                const int base = (seen >> 4) == prm.split_epoch ? seen : (prm.split_epoch << 4);
                if (__hip_atomic_compare_exchange_strong(&tickets[0], &seen, base + 1, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                         __HIP_MEMORY_SCOPE_AGENT)) {
                    note[0] = base & 15;
                    break;
                }
            }
        }
        __syncthreads();
        if (note[0] < parts - 1) {
            float* record = records + part * kSplitRecordFloats;
#pragma unroll
            for (int dt = 0; dt < 4; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    __hip_atomic_store(record + (16 * dt + r) * kPfThreads, o[0][dt][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(record + 64 * kPfThreads, m_run[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(record + 65 * kPfThreads, l_run[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            wait_vm<0>();                            // the stores have been acknowledged
            __syncthreads();
            // Publication order without a release fence: every store of the record is an agent-scope atomic store
            // (written through to where every XCD of the device reads it), each wave has waited for the
            // acknowledgement of its own stores (vmcnt 0) before the block barrier above, and the flag, which
            // carries the launch's epoch, is stored after that barrier.  A release on the flag would add a
            // write-back of every dirty line of this XCD's L2 (the output rows and cache pages of all the blocks
            // that run beside this one) in front of it: measured 25.2 us against 20.3 us for one prompt of 1024
            // tokens, with nothing in the record left for that write-back to publish.
            if (tid == 0) __hip_atomic_store(&tickets[1 + part], prm.split_epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return;
        }
        if (tid == 0) {
            // the publishers drew their tickets before this block and are running: short waits, bounded all the same
            unsigned spins = 0;
            for (int p = 0; p < parts; ++p) {
                if (p == part) continue;
                while (__hip_atomic_load(&tickets[1 + p], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) != prm.split_epoch
                       && spins < kSplitSpinLimit) {
                    __builtin_amdgcn_s_sleep(2);
                    ++spins;
                }
            }
            note[1] = spins < kSplitSpinLimit ? 1 : 0;
            // Back to zero: a captured launch is replayed with the epoch it was captured with and must find no
            // arrivals of its own number.  (After a wait that gave up a late flag may survive this; launches
            // with another epoch ignore it, a replay of the same captured launch needs the workspace
            // initialised again, which is what QM_STATUS_SPLIT_TIMEOUT asks for.)
            for (int i = 0; i <= parts; ++i)
                __hip_atomic_store(&tickets[i], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        if (note[1] == 0) {
            if (tid == 0 && prm.status) atomicOr(prm.status, QM_STATUS_SPLIT_TIMEOUT);
            return;
        }
        float m_part[kSplitMaxParts], w_part[kSplitMaxParts];
        float m_all = -INFINITY;
#pragma unroll
        for (int p = 0; p < kSplitMaxParts; ++p) {
            m_part[p] = -INFINITY;
            if (p < parts)
                m_part[p] = p == part ? m_run[0]
                          : __hip_atomic_load(records + p * kSplitRecordFloats + 64 * kPfThreads, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            m_all = fmaxf(m_all, m_part[p]);
        }
        float l_all = 0.0f;
#pragma unroll
        for (int p = 0; p < kSplitMaxParts; ++p) {
            w_part[p] = m_part[p] == -INFINITY ? 0.0f : fast_exp2((m_part[p] - m_all) * coef);
            if (p < parts) {
                const float l_p = p == part ? l_run[0]
                                : __hip_atomic_load(records + p * kSplitRecordFloats + 65 * kPfThreads, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                l_all = p == 0 ? l_p * w_part[p] : l_all + l_p * w_part[p];
            }
        }
        l_run[0] = l_all;
        // (two of the four d tiles at a time: every record load of a round is in flight before the first is used;
        // the other parts' values sit in three slots, part p in slot p or p - 1, whichever skips this block's own)
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            float term[kSplitMaxParts - 1][32];
#pragma unroll
            for (int j = 0; j < kSplitMaxParts - 1; ++j) {
                if (j >= parts - 1) continue;
                const float* src = records + (j < part ? j : j + 1) * kSplitRecordFloats + 32 * half * kPfThreads;
#pragma unroll
                for (int i = 0; i < 32; ++i)
                    term[j][i] = __hip_atomic_load(src + i * kPfThreads, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                float sum = 0.0f;
#pragma unroll
                for (int p = 0; p < kSplitMaxParts; ++p) {
                    if (p >= parts) continue;
                    float x = o[0][2 * half + i / 16][i % 16];
                    if (p < part && p < kSplitMaxParts - 1) x = term[p < kSplitMaxParts - 1 ? p : 0][i];
                    if (p > part) x = term[p > 0 ? p - 1 : 0][i];
                    x *= w_part[p];
                    sum = p == 0 ? x : sum + x;
                }
                o[0][2 * half + i / 16][i % 16] = sum;
            }
        }
        __syncthreads();                             // the notes have been read: the area is the staging area again
    }

    // ---- normalise and write, straight from the registers: no staging area, so a wave that is done does not wait
    // for the others.  A lane holds dims 32 dt + 8 rq + 4 grp .. + 3 of its column; the two halves of the wave
    // exchange (v_permlane32_swap) so that the lower half owns the eight dims of even rq and the upper half those of
    // odd rq: 16 bytes per lane, 32 contiguous bytes per row and request. ----
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const float l_tot = halves_sum(l_run[c]);
        const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
        const int row = group_row0(c) + (col & 15);
        uint16_t* dst = prm.out + ((static_cast<int64_t>(b) * S + row) * q_heads + my_head) * kDim + 8 * grp;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) {
#pragma unroll
            for (int rp = 0; rp < 2; ++rp) {
                const int re = 8 * rp;               // registers of rq = 2 rp (even) and + 4 (odd)
                const uint32_t e0 = pack_bf16_pair(o[c][dt][re + 0] * inv, o[c][dt][re + 1] * inv);
                const uint32_t e1 = pack_bf16_pair(o[c][dt][re + 2] * inv, o[c][dt][re + 3] * inv);
                const uint32_t o0 = pack_bf16_pair(o[c][dt][re + 4] * inv, o[c][dt][re + 5] * inv);
                const uint32_t o1 = pack_bf16_pair(o[c][dt][re + 6] * inv, o[c][dt][re + 7] * inv);
                // lower half: (e, e of the partner); upper half: (o of the partner, o)
                const auto x = __builtin_amdgcn_permlane32_swap(e0, o0, false, false);
                const auto y = __builtin_amdgcn_permlane32_swap(e1, o1, false, false);
                const uint4 val = make_uint4(x[0], y[0], x[1], y[1]);
                if (row < S) *reinterpret_cast<uint4*>(dst + 32 * dt + 16 * rp) = val;
            }
        }
    }
}

// grid = batch * kv_heads * ceil(seq / (64 NC)) blocks.  Blocks of the first query tile run the uniform-waves body
// on its one or two 64-row tiles (split-precision P in the very first).
template <bool ROUND, int NC>
__global__ __launch_bounds__(kPfThreads, (NC == 1 ? 2 : 1)) void prefill_il_kernel(PrefillParams prm, qm_kv_cache cache) {
    extern __shared__ __attribute__((aligned(16))) unsigned char il_smem[];
    request_arguments(prm, cache);
    const int pairs = prm.batch * prm.kv_heads;
    const int bid = blockIdx.x;
    // Heaviest query tile first; when the whole grid is resident at once (at most two blocks per CU,
    // the second block of a CU being the one CUs later in the grid) the blocks after the first `CUs`
    // ascend from the lightest tile, so that a CU's two blocks are a heavy and a light one.
    const int group = bid / pairs;
    // key split: the blocks of a query tile's parts follow one another, heaviest query tile first
    int qt, part = 0, parts = 1;
    if (NC == 1 && prm.split_chunk > 0) {
        int left = group;
        for (qt = prm.n_qtiles - 1; qt > 0; --qt) {
            parts = split_parts(qt + 1, prm.split_chunk);
            if (left < parts) break;
            left -= parts;
        }
        part = qt > 0 ? left : 0;
        parts = qt > 0 ? parts : 1;
    } else {
        qt = group < prm.heavy_groups ? prm.n_qtiles - 1 - group : group - prm.heavy_groups;
    }
    if (qt == 0) {
        const int pair = bid % pairs;
        // (with the whole grid resident the lightest block also writes the pages of the last key tiles: the blocks
        // of the heavier half write none)
        if (prm.has_cache != 0 && prm.dealt_pages != 0) {
#pragma unroll 1
            for (int j = 0; j < kHeavyTilesPerBlock; ++j) {
                const int heavy = prm.n_qtiles - 1 - j;
                if (heavy >= prm.n_qtiles - prm.n_qtiles / 2) copy_tile_to_pages(prm, cache, pair / prm.kv_heads, pair % prm.kv_heads, heavy);
            }
        }
        prefill_body<true, ROUND>(prm, cache, il_smem, 0, pair);
    } else {
        prefill_il_body<ROUND, NC>(prm, cache, il_smem, qt, bid % pairs, part, parts, prm.n_qtiles - 1 - qt);
    }
}

// Sets the tickets of a key-split workspace to zero (a kernel, not a memset: callers may capture it).
__global__ void prefill_split_clear_kernel(int* tickets, int64_t count) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < count) tickets[i] = 0;
}

// The key split of a call: how long a run of key tiles a block takes, and the workspace that takes.
struct SplitPlan {
    int chunk = 0;               // 0: no split
    int slots = 0;               // split query tiles per pair
    int64_t groups = 0;          // blocks per pair
    int64_t ticket_bytes = 0;    // rounded up to 256
    int64_t bytes = 0;           // tickets + records
};

// Split when the grid stays resident at once with the added blocks: then the kernel lasts as long as the longest
// chain and the chip has room for more blocks.  The shortest run of key tiles is taken with which every block still
// has a CU to itself, else the shortest with at most two blocks per CU (beyond that the added blocks would have
// to wait for a CU and the split loses: a block spends 12 000 to 16 000 cycles outside its pipeline, about six key
// tiles' worth; measured 4 x 1024: 32 us whole, 41 us in halves).  Publishing, waiting and combining cost about
// as much as three key tiles (measured: runs of four on 384 tokens 14.2 us against 13.4 us whole): runs are six
// key tiles at least and the longest chain has to drop by three.
static SplitPlan plan_split(int64_t pairs, int seq, int compute_units) {
    SplitPlan plan;
    const int n_qtiles = (seq + kBM - 1) / kBM;
    for (int per_cu = 1; per_cu <= 2 && plan.chunk == 0; ++per_cu) {
        for (int chunk = 6; chunk + 3 <= n_qtiles; ++chunk) {
            int64_t groups = 0;
            for (int qt = 0; qt < n_qtiles; ++qt) groups += split_parts(qt + 1, chunk);
            if (pairs * groups > per_cu * static_cast<int64_t>(compute_units)) continue;
            plan.chunk = chunk;
            plan.slots = n_qtiles - chunk;                    // query tiles of more than `chunk` key tiles
            plan.groups = groups;
            // (tickets take the same room for every shape, that of the most split query tiles a resident grid can
            // hold: a workspace that has served one shape holds no record where another shape keeps tickets)
            const int64_t items = pairs * plan.slots;
            plan.ticket_bytes = (2 * static_cast<int64_t>(compute_units) * kSplitTicketInts * static_cast<int64_t>(sizeof(int)) + 255) / 256 * 256;
            plan.bytes = plan.ticket_bytes + items * kSplitMaxParts * kSplitRecordFloats * static_cast<int64_t>(sizeof(float));
            break;
        }
    }
    return plan;
}

static int32_t device_compute_units(int* compute_units) {
    int device = 0;
    hipError_t err = hipGetDevice(&device);
    if (err == hipSuccess) err = hipDeviceGetAttribute(compute_units, hipDeviceAttributeMultiprocessorCount, device);
    return err == hipSuccess ? QM_OK : hip_code(err);
}

}  // namespace qm


extern "C" int64_t qm_prefill_split_workspace_bytes(int32_t batch, int32_t seq, int32_t kv_heads) {
    using namespace qm;
    if (batch <= 0 || seq <= 0 || kv_heads <= 0) return 0;
    int compute_units = 0;
    const int32_t rc = device_compute_units(&compute_units);
    if (rc != QM_OK) return rc;
    return plan_split(static_cast<int64_t>(batch) * kv_heads, seq, compute_units).bytes;
}

extern "C" int32_t qm_prefill_split_workspace_init(void* workspace, int64_t workspace_bytes, void* hip_stream) {
    using namespace qm;
    if (workspace_bytes < 0) return QM_ERR_ARGUMENT;
    if (workspace_bytes == 0) return QM_OK;
    if (!workspace) return QM_ERR_NULL;
    if (reinterpret_cast<uintptr_t>(workspace) & 255) return QM_ERR_GEOMETRY;
    // tickets lie in front of the records; clearing the whole area is the simple rule that needs no geometry
    const int64_t count = workspace_bytes / static_cast<int64_t>(sizeof(int));
    const int64_t blocks = (count + 255) / 256;
    if (blocks > 0x7fffffffLL) return QM_ERR_ARGUMENT;
    hipLaunchKernelGGL(prefill_split_clear_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       static_cast<hipStream_t>(hip_stream), static_cast<int*>(workspace), count);
    return launch_status();
}

static int32_t prefill_attention_entry(
    const uint16_t* query, const uint16_t* key, const uint16_t* value,
    uint16_t* context_out,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    int32_t batch, int32_t seq, int32_t q_heads, int32_t kv_heads, float scale,
    int64_t kv_stride_token, int64_t kv_stride_head, int64_t kv_stride_batch,
    void* workspace, int64_t workspace_bytes,
    uint32_t* status_dev, void* hip_stream) {
    using namespace qm;
    if (workspace_bytes < 0 || (workspace_bytes > 0 && !workspace)) return QM_ERR_ARGUMENT;
    if (reinterpret_cast<uintptr_t>(workspace) & 255) return QM_ERR_GEOMETRY;
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
    prm.heavy_groups = n_qtiles;
    prm.dealt_pages = 0;
    prm.split_chunk = 0; prm.split_slots = 0; prm.split_partials = nullptr; prm.split_tickets = nullptr; prm.split_epoch = 0;
    prm.cache_before = 0; prm.key_count = seq;

    hipStream_t s = static_cast<hipStream_t>(hip_stream);
    const bool round_scores = option_value(QM_OPT_PREFILL_SCORE_ROUNDING) != 0;
    if (!round_scores && !(scale > 0.0f)) return QM_ERR_ARGUMENT;   // the scale is folded into the exponent there
    // 0: the interleaved waves (fastest at every size measured); 1: the uniform waves
    const int which = option_value(QM_OPT_PREFILL_KERNEL);
    if (which < 0 || which > 1) return QM_ERR_ARGUMENT;
    // (its running maximum is taken before the scores are scaled: a negative scale goes to the uniform waves)
    if (which == 0 && scale >= 0.0f) {
        int compute_units = 0;
        const int32_t rc_cu = device_compute_units(&compute_units);
        if (rc_cu != QM_OK) return rc_cu;
        int64_t blocks = pairs * prm.n_qtiles;
        const SplitPlan split = workspace ? plan_split(pairs, seq, compute_units) : SplitPlan();
        if (split.chunk > 0) {
            if (workspace_bytes < split.bytes) return QM_ERR_WORKSPACE;
            static std::atomic<uint32_t> launches{0};
            prm.split_epoch = static_cast<int>(launches.fetch_add(1, std::memory_order_relaxed) % 0x7FFFFFEu) + 1;
            prm.split_chunk = split.chunk;
            prm.split_slots = split.slots;
            prm.split_tickets = static_cast<int*>(workspace);
            prm.split_partials = reinterpret_cast<float*>(static_cast<unsigned char*>(workspace) + split.ticket_bytes);
            blocks = pairs * split.groups;
        } else if (compute_units % pairs == 0 && blocks > compute_units && blocks <= 2 * static_cast<int64_t>(compute_units)) {
            prm.heavy_groups = static_cast<int>(compute_units / pairs);
        }
        prm.dealt_pages = blocks <= 2 * static_cast<int64_t>(compute_units) ? 1 : 0;   // two blocks fit a CU
        static std::atomic<bool> lds_raised[2][kMaxDevices];
        const void* kernel = round_scores ? reinterpret_cast<const void*>(prefill_il_kernel<true, 1>)
                                          : reinterpret_cast<const void*>(prefill_il_kernel<false, 1>);
        const int32_t rc_lds = ensure_dynamic_lds(kernel, kIlSmemBytes, lds_raised[round_scores ? 1 : 0]);
        if (rc_lds != QM_OK) return rc_lds;
        const dim3 grid(static_cast<unsigned>(blocks));
        if (round_scores) hipLaunchKernelGGL((prefill_il_kernel<true, 1>), grid, dim3(kPfThreads), kIlSmemBytes, s, prm, desc);
        else hipLaunchKernelGGL((prefill_il_kernel<false, 1>), grid, dim3(kPfThreads), kIlSmemBytes, s, prm, desc);
        return launch_status();
    }
    const size_t smem = sizeof(PfStage) * kPfStages;
    const auto kernel = round_scores ? prefill_causal_kernel<true> : prefill_causal_kernel<false>;
    static std::atomic<bool> lds_raised[2][kMaxDevices];
    const int32_t rc_lds = ensure_dynamic_lds(reinterpret_cast<const void*>(kernel), static_cast<int>(smem),
                                              lds_raised[round_scores ? 1 : 0]);
    if (rc_lds != QM_OK) return rc_lds;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(pairs * n_qtiles)), dim3(kPfThreads), smem, s, prm, desc);
    return launch_status();
}


extern "C" int32_t qm_prefill_attention_causal(
    const uint16_t* query, const uint16_t* key, const uint16_t* value,
    uint16_t* context_out,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    int32_t batch, int32_t seq, int32_t q_heads, int32_t kv_heads, float scale,
    int64_t kv_stride_token, int64_t kv_stride_head, int64_t kv_stride_batch,
    uint32_t* status_dev, void* hip_stream) {
    return prefill_attention_entry(query, key, value, context_out, cache, page_table, max_pages, batch, seq, q_heads,
                                   kv_heads, scale, kv_stride_token, kv_stride_head, kv_stride_batch, nullptr, 0,
                                   status_dev, hip_stream);
}

extern "C" int32_t qm_prefill_attention_causal_split(
    const uint16_t* query, const uint16_t* key, const uint16_t* value,
    uint16_t* context_out,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    int32_t batch, int32_t seq, int32_t q_heads, int32_t kv_heads, float scale,
    int64_t kv_stride_token, int64_t kv_stride_head, int64_t kv_stride_batch,
    void* workspace, int64_t workspace_bytes,
    uint32_t* status_dev, void* hip_stream) {
    return prefill_attention_entry(query, key, value, context_out, cache, page_table, max_pages, batch, seq, q_heads,
                                   kv_heads, scale, kv_stride_token, kv_stride_head, kv_stride_batch, workspace,
                                   workspace_bytes, status_dev, hip_stream);
}

namespace qm {

// The key split of a chunk call: with fewer blocks than compute units the key tiles of a query tile are handed out in
// runs, as many per query tile as fill the chip, of four tiles at least and sixteen runs at most.
struct ChunkPlan {
    int parts = 1;       // blocks per (pair, query tile)
    int run = 0;         // key tiles per block
    int64_t bytes = 0;   // records
};

static ChunkPlan plan_chunk(int64_t pairs, int rows, int cache_before, int compute_units, int gqa_group) {
    ChunkPlan plan;
    const int block_rows = 128 / gqa_group;
    const int n_qtiles = (rows + block_rows - 1) / block_rows;
    const int64_t blocks = pairs * n_qtiles;
    const int tiles = (cache_before + rows - 1) / kBN + 1;      // of the last query tile
    int64_t parts = (compute_units + blocks - 1) / blocks;
    parts = std::min<int64_t>(parts, std::min(tiles / 4, kChunkMaxRuns));
    if (parts < 2) return plan;
    plan.run = static_cast<int>((tiles + parts - 1) / parts);
    plan.parts = (tiles + plan.run - 1) / plan.run;
    if (plan.parts < 2) return ChunkPlan();
    plan.bytes = blocks * plan.parts * kChunkRecordFloats * static_cast<int64_t>(sizeof(float));
    return plan;
}

static bool chunk_group_served(int32_t q_heads, int32_t kv_heads) {
    return kv_heads > 0 && (q_heads == kv_heads || q_heads == 2 * kv_heads || q_heads == 4 * kv_heads);
}

template <int G>
static int32_t launch_chunk_kernels(const PrefillParams& prm, const qm_kv_cache& cache, bool round_scores, int64_t pairs, hipStream_t s) {
    const size_t smem = sizeof(PfStage) * kPfStages;
    const auto kernel = round_scores ? prefill_chunk_kernel<true, G> : prefill_chunk_kernel<false, G>;
    static std::atomic<bool> lds_raised[2][kMaxDevices];
    const int32_t rc_lds = ensure_dynamic_lds(reinterpret_cast<const void*>(kernel), static_cast<int>(smem),
                                              lds_raised[round_scores ? 1 : 0]);
    if (rc_lds != QM_OK) return rc_lds;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(pairs * prm.n_qtiles * prm.chunk_parts)), dim3(kPfThreads), smem, s, prm, cache);
    int32_t rc = launch_status();
    if (rc == QM_OK && prm.chunk_parts > 1) {
        hipLaunchKernelGGL(prefill_chunk_merge_kernel, dim3(static_cast<unsigned>(pairs * prm.n_qtiles * kChunkMergeSlices)), dim3(kPfThreads), 0, s,
                           prm, round_scores ? 1 : 0, G);
        rc = launch_status();
    }
    return rc;
}

// What the two chunk entry points share once the keys' addressing is settled in `prm` / `cache`.
static int32_t chunk_entry(PrefillParams& prm, const qm_kv_cache& cache, int32_t batch, int32_t rows, int32_t cache_before,
                           int32_t q_heads, int32_t kv_heads, float scale, void* workspace, int64_t workspace_bytes, void* hip_stream) {
    const int gqa_group = q_heads / kv_heads;
    const int block_rows = 128 / gqa_group;
    const int n_qtiles = (rows + block_rows - 1) / block_rows;
    const int64_t pairs = static_cast<int64_t>(batch) * kv_heads;
    if (pairs * n_qtiles * 16 > 0x7fffffffLL) return QM_ERR_ARGUMENT;
    prm.batch = batch; prm.seq = rows; prm.kv_heads = kv_heads; prm.n_qtiles = n_qtiles; prm.scale = scale;
    prm.heavy_groups = n_qtiles;
    prm.dealt_pages = 0;
    prm.cache_before = cache_before; prm.key_count = cache_before + rows;
    prm.chunk_parts = 1;
    if (workspace) {
        int compute_units = 0;
        const int32_t rc_cu = device_compute_units(&compute_units);
        if (rc_cu != QM_OK) return rc_cu;
        const ChunkPlan plan = plan_chunk(pairs, rows, cache_before, compute_units, gqa_group);
        if (plan.parts > 1) {
            if (workspace_bytes < plan.bytes) return QM_ERR_WORKSPACE;
            prm.chunk_parts = plan.parts;
            prm.chunk_run = plan.run;
            prm.chunk_records = static_cast<float*>(workspace);
        }
    }
    const bool round_scores = option_value(QM_OPT_PREFILL_SCORE_ROUNDING) != 0;
    if (!round_scores && !(scale > 0.0f)) return QM_ERR_ARGUMENT;   // the scale is folded into the exponent there
    hipStream_t s = static_cast<hipStream_t>(hip_stream);
    if (gqa_group == 1) return launch_chunk_kernels<1>(prm, cache, round_scores, pairs, s);
    if (gqa_group == 2) return launch_chunk_kernels<2>(prm, cache, round_scores, pairs, s);
    return launch_chunk_kernels<4>(prm, cache, round_scores, pairs, s);
}

}  // namespace qm

extern "C" int64_t qm_prefill_chunk_workspace_bytes(int32_t batch, int32_t rows, int32_t cache_before, int32_t kv_heads) {
    using namespace qm;
    if (batch <= 0 || rows <= 0 || cache_before < 0 || kv_heads <= 0) return 0;
    if (static_cast<int64_t>(cache_before) + rows > INT32_MAX) return QM_ERR_ARGUMENT;
    int compute_units = 0;
    const int32_t rc = device_compute_units(&compute_units);
    if (rc != QM_OK) return rc;
    // (enough for any of the groups served: the smaller the group, the fewer and longer the query tiles)
    int64_t bytes = 0;
    for (int g = 1; g <= 4; g *= 2)
        bytes = std::max(bytes, plan_chunk(static_cast<int64_t>(batch) * kv_heads, rows, cache_before, compute_units, g).bytes);
    return bytes;
}

extern "C" int32_t qm_prefill_attention_chunk(
    const uint16_t* query, const uint16_t* key, const uint16_t* value,
    uint16_t* context_out,
    int32_t batch, int32_t rows, int32_t cache_before, int32_t q_heads, int32_t kv_heads, float scale,
    int64_t kv_stride_token, int64_t kv_stride_head, int64_t kv_stride_batch,
    void* workspace, int64_t workspace_bytes,
    void* hip_stream) {
    using namespace qm;
    if (batch < 0 || rows < 0 || cache_before < 0) return QM_ERR_ARGUMENT;
    if (workspace_bytes < 0 || (workspace_bytes > 0 && !workspace)) return QM_ERR_ARGUMENT;
    if (reinterpret_cast<uintptr_t>(workspace) & 255) return QM_ERR_GEOMETRY;
    const int64_t key_count = static_cast<int64_t>(cache_before) + rows;
    if (kv_stride_token == 0 && kv_stride_head == 0 && kv_stride_batch == 0) {
        kv_stride_token = static_cast<int64_t>(kv_heads) * kDim;     // [batch][key_count][kv_heads][128]
        kv_stride_head = kDim;
        kv_stride_batch = key_count * kv_heads * kDim;
    }
    if (kv_stride_token < kDim || kv_stride_head < 0 || kv_stride_batch < 0
        || ((kv_stride_token | kv_stride_head | kv_stride_batch) & 7))
        return QM_ERR_GEOMETRY;
    if (key_count * kv_stride_token >= (1LL << 31)) return QM_ERR_ARGUMENT;
    if (!query || !key || !value || !context_out) return QM_ERR_NULL;
    if (!chunk_group_served(q_heads, kv_heads)) return QM_ERR_GEOMETRY;     // 32 / G query rows x G heads on the MFMA columns
    const uintptr_t align = reinterpret_cast<uintptr_t>(query) | reinterpret_cast<uintptr_t>(key)
                          | reinterpret_cast<uintptr_t>(value) | reinterpret_cast<uintptr_t>(context_out);
    if (align & 15) return QM_ERR_GEOMETRY;
    if (batch == 0 || rows == 0) return QM_OK;
    PrefillParams prm = {};
    prm.q = query; prm.k = key; prm.v = value; prm.out = context_out;
    prm.pages = make_page_map(16, 1);
    prm.kv_stride_token = kv_stride_token; prm.kv_stride_head = kv_stride_head; prm.kv_stride_batch = kv_stride_batch;
    const qm_kv_cache none = {};
    return chunk_entry(prm, none, batch, rows, cache_before, q_heads, kv_heads, scale, workspace, workspace_bytes, hip_stream);
}

extern "C" int32_t qm_prefill_attention_chunk_paged(
    const uint16_t* query, const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    uint16_t* context_out,
    int32_t batch, int32_t rows, int32_t cache_before, int32_t q_heads, int32_t kv_heads, float scale,
    void* workspace, int64_t workspace_bytes, uint32_t* status_dev,
    void* hip_stream) {
    using namespace qm;
    if (batch < 0 || rows < 0 || cache_before < 0) return QM_ERR_ARGUMENT;
    if (workspace_bytes < 0 || (workspace_bytes > 0 && !workspace)) return QM_ERR_ARGUMENT;
    if (reinterpret_cast<uintptr_t>(workspace) & 255) return QM_ERR_GEOMETRY;
    if (!query || !context_out || !page_table) return QM_ERR_NULL;
    const int32_t rc = check_cache(cache, max_pages);
    if (rc != QM_OK) return rc;
    if (cache->kv_heads != kv_heads || !chunk_group_served(q_heads, kv_heads)) return QM_ERR_GEOMETRY;
    if (cache->page_size % 16) return QM_ERR_GEOMETRY;              // a 16-key group lies in one page
    const int64_t key_count = static_cast<int64_t>(cache_before) + rows;
    if (key_count > cache_capacity(cache, max_pages) || key_count > INT32_MAX) return QM_ERR_SLOT_RANGE;
    if ((reinterpret_cast<uintptr_t>(query) | reinterpret_cast<uintptr_t>(context_out)) & 15) return QM_ERR_GEOMETRY;
    if (batch == 0 || rows == 0) return QM_OK;
    PrefillParams prm = {};
    prm.q = query; prm.out = context_out;
    prm.k = cache->k_pool; prm.v = cache->v_pool;                   // (not read: the tiles come through the page table)
    prm.pages = make_page_map(cache->page_size, max_pages);
    prm.kv_stride_token = kDim; prm.kv_stride_head = 0; prm.kv_stride_batch = 0;
    prm.chunk_table = page_table; prm.chunk_paged = 1;
    prm.status = status_dev;
    return chunk_entry(prm, *cache, batch, rows, cache_before, q_heads, kv_heads, scale, workspace, workspace_bytes, hip_stream);
}
