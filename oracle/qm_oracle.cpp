// qm_oracle.cpp — TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// Scalar CPU restatement (fp32 accumulate, bf16 storage) of the attention / KV-cache
// operators of the reference engine, devices/rx7900xtx-24g/qwen3_tts_1_7b.cpp ("R17").
// Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load this
// library; the shipped library (libqm_attn.so) never links or calls it.
//
// The reference has no CPU implementation and ships no golden vectors for this path,
// so every function here follows the reference *source text* line by line (cited at
// each function) and is pinned by the closed forms / invariants / brute-force checks
// in tests/test_oracle_*.py.  What cannot be pinned here: agreement of the reference's
// bf16 boundary chain with upstream PyTorch on real weights (claimed in the comments at
// R17:15446, 15879) — parity unpinned against upstream, inherited as an assumption.
//
// Device-specific arithmetic that has no bit-exact CPU twin is restated as follows:
//   rsqrtf(x)  (R17:15437, 12198, 8309)  ->  1.0f / sqrtf(x), both correctly rounded;
//   expf(x)    (R17:15933, 12490, 9582)  ->  glibc expf.
// Wave32 shuffle-tree reductions (R17:15059-15148, 8233-8274, 9358-9364) are simulated
// lane by lane so that fp32 summation order is the reference's.
//
// Attention policies (last argument of the attention functions):
//   QMO_POLICY_REFERENCE  the reference chain: bf16(QK) -> bf16(*scale) -> fp32 softmax
//                         -> bf16(P) -> fp32 P.V -> bf16            (R17:15841-16005)
//   QMO_POLICY_ONLINE     same score roundings; P stays fp32 and is normalised after the
//                         P.V accumulation (what an online-softmax kernel computes)
//   QMO_POLICY_FP32       no intermediate rounding at all (plain softmax(QK^T*scale)V)

#include <cmath>
#include <cstdint>
#include <cstring>
#include <thread>
#include <vector>
#include <algorithm>
#include <functional>

#include "../include/qm_attn.h"

#define QMO_POLICY_REFERENCE 0
#define QMO_POLICY_ONLINE    1
#define QMO_POLICY_FP32      2

namespace {

constexpr int kDim = 128;

// R17:15024-15031
inline float bf2f(uint16_t v) {
    uint32_t bits = static_cast<uint32_t>(v) << 16;
    float f;
    std::memcpy(&f, &bits, sizeof f);
    return f;
}

// R17:15034-15056 (same as 79-101, 8172-8187, host 21570-21574)
inline uint16_t f2bf(float value) {
    uint32_t bits;
    std::memcpy(&bits, &value, sizeof bits);
    if ((bits & 0x7fffffffU) > 0x7f800000U) {
        return static_cast<uint16_t>((bits >> 16) | 0x0040U);
    }
    const uint32_t lsb = (bits >> 16) & 1U;
    bits += 0x7fffU + lsb;
    return static_cast<uint16_t>(bits >> 16);
}

// value += __shfl_down(value, offset) for offset 16..1 on a 32-lane wave; a lane whose
// source is out of range receives its own value (R17:15059-15075, 9358-9364).
// Returns lane 0.
inline float wave32_sum(const float* lanes) {
    // Only the lanes that feed lane 0 matter; all of their sources are in range.
    float a[16], b[8], c[4], d[2];
    for (int i = 0; i < 16; ++i) a[i] = lanes[i] + lanes[i + 16];
    for (int i = 0; i < 8; ++i) b[i] = a[i] + a[i + 8];
    for (int i = 0; i < 4; ++i) c[i] = b[i] + b[i + 4];
    for (int i = 0; i < 2; ++i) d[i] = c[i] + c[i + 2];
    return d[0] + d[1];
}

// R17:15078-15099: value = value > other ? value : other.
inline float wave32_max(const float* lanes) {
    auto mx = [](float v, float o) { return v > o ? v : o; };
    float a[16], b[8], c[4], d[2];
    for (int i = 0; i < 16; ++i) a[i] = mx(lanes[i], lanes[i + 16]);
    for (int i = 0; i < 8; ++i) b[i] = mx(a[i], a[i + 8]);
    for (int i = 0; i < 4; ++i) c[i] = mx(b[i], b[i + 4]);
    for (int i = 0; i < 2; ++i) d[i] = mx(c[i], c[i + 2]);
    return mx(d[0], d[1]);
}

// talker_block_sum / talker_block_max over `threads` per-thread values
// (R17:15102-15197): wave trees, then a tree over the per-wave results in wave 0.
inline float block_sum(const float* per_thread, int threads) {
    const int waves = (threads + 31) >> 5;
    float wave_values[32];
    for (int w = 0; w < 32; ++w) wave_values[w] = 0.0f;
    for (int w = 0; w < waves; ++w) {
        float lanes[32];
        for (int l = 0; l < 32; ++l) {
            const int t = w * 32 + l;
            lanes[l] = t < threads ? per_thread[t] : 0.0f;
        }
        wave_values[w] = wave32_sum(lanes);
    }
    return wave32_sum(wave_values);
}

inline float block_max(const float* per_thread, int threads) {
    const int waves = (threads + 31) >> 5;
    float wave_values[32];
    for (int w = 0; w < 32; ++w) wave_values[w] = -INFINITY;
    for (int w = 0; w < waves; ++w) {
        float lanes[32];
        for (int l = 0; l < 32; ++l) {
            const int t = w * 32 + l;
            lanes[l] = t < threads ? per_thread[t] : -INFINITY;
        }
        wave_values[w] = wave32_max(lanes);
    }
    return wave32_max(wave_values);
}

// Sum of squares of one 128-wide head in the reference's order: one thread per
// dimension, x*x, 32-lane trees, then the tree over the four wave sums
// (R17:15429-15433 with 128 threads; R17:12178-12194 and 8292-8304 with 256 threads,
// whose upper four waves contribute exact zeros — same result).
inline float head_sum_squares(const uint16_t* x) {
    float sq[kDim];
    for (int d = 0; d < kDim; ++d) {
        const float v = bf2f(x[d]);
        sq[d] = v * v;
    }
    return block_sum(sq, kDim);
}

inline float inverse_rms(float sum, float epsilon) {
    // R17:15436-15441: rsqrtf(sum / head_dim + epsilon)
    return 1.0f / std::sqrt(sum / static_cast<float>(kDim) + epsilon);
}

// RMSNorm of one head: bf16(x*r) then bf16(that * gamma)   (R17:15448-15460, 8321-8336)
inline void head_rmsnorm(const uint16_t* x, const uint16_t* gamma, float epsilon,
                         uint16_t* out) {
    const float r = inverse_rms(head_sum_squares(x), epsilon);
    for (int d = 0; d < kDim; ++d) {
        const uint16_t n = f2bf(bf2f(x[d]) * r);
        out[d] = f2bf(bf2f(n) * bf2f(gamma[d]));
    }
}

// RoPE of one head: bf16(bf16(x*cos) + bf16(rotate_half(x)*sin)), rotate_half = (-x2, +x1)
// (R17:15464-15498, 15571-15624, 8432-8488)
inline void head_rope(const uint16_t* x, const uint16_t* cosv, const uint16_t* sinv,
                      uint16_t* out) {
    uint16_t tmp[kDim];
    for (int d = 0; d < kDim; ++d) {
        const int rd = d < kDim / 2 ? d + kDim / 2 : d - kDim / 2;
        float rotated = bf2f(x[rd]);
        if (d < kDim / 2) rotated = -rotated;
        const uint16_t first = f2bf(bf2f(x[d]) * bf2f(cosv[d]));
        const uint16_t second = f2bf(rotated * bf2f(sinv[d]));
        tmp[d] = f2bf(bf2f(first) + bf2f(second));
    }
    std::memcpy(out, tmp, sizeof tmp);
}

// Element offset of (token, head) in the paged pool; -1 if out of range.
inline int64_t slot_offset(const qm_kv_cache* c, const int32_t* page_table,
                           int32_t max_pages, int64_t token, int head) {
    if (token < 0) return -1;
    const int64_t page = token / c->page_size;
    if (page >= max_pages) return -1;
    const int64_t phys = page_table ? page_table[page] : page;
    if (phys < 0 || phys >= c->n_pages) return -1;
    return phys * c->stride_page + static_cast<int64_t>(head) * c->stride_head
         + (token % c->page_size) * c->stride_token;
}

// One score: the reference's wave-per-key dot product — lane l accumulates dims
// l, l+32, l+64, l+96 with fmaf, then the 32-lane tree (R17:15850-15876, 16080-16100,
// 9434-9454, 12386-12418).
inline float qk_dot(const uint16_t* q, const uint16_t* k) {
    float lanes[32];
    for (int l = 0; l < 32; ++l) {
        float acc = 0.0f;
        for (int d = l; d < kDim; d += 32) acc = std::fmaf(bf2f(q[d]), bf2f(k[d]), acc);
        lanes[l] = acc;
    }
    return wave32_sum(lanes);
}

inline float score_from_dot(float acc, float scale, int policy) {
    if (policy == QMO_POLICY_FP32) return acc * scale;
    // R17:15881-15890: bf16(acc), then bf16(that * scale)
    const uint16_t raw = f2bf(acc);
    return bf2f(f2bf(bf2f(raw) * scale));
}

using RowPtr = std::function<const uint16_t*(int)>;

// Attention of one query head vector over keys [key_start, key_end) in the talker's
// topology: 256 threads, thread-strided softmax partials, serial P.V
// (R17:15894-16005 == 16121-16202).
void attend_talker(const uint16_t* q, const RowPtr& key_row, const RowPtr& value_row,
                   int key_start, int key_end, float scale, int policy, uint16_t* out) {
    const int n = key_end - key_start;
    if (n <= 0) {
        for (int d = 0; d < kDim; ++d) out[d] = 0;
        return;
    }
    std::vector<float> s(n);
    for (int i = 0; i < n; ++i) {
        s[i] = score_from_dot(qk_dot(q, key_row(key_start + i)), scale, policy);
    }
    if (policy == QMO_POLICY_REFERENCE) {
        constexpr int T = 256;
        float part[T];
        for (int t = 0; t < T; ++t) {
            float m = -INFINITY;
            for (int i = t; i < n; i += T) m = m > s[i] ? m : s[i];
            part[t] = m;
        }
        const float maximum = block_max(part, T);
        for (int t = 0; t < T; ++t) {
            float acc = 0.0f;
            for (int i = t; i < n; i += T) acc += std::exp(s[i] - maximum);
            part[t] = acc;
        }
        const float total = block_sum(part, T);
        std::vector<float> p(n);
        for (int i = 0; i < n; ++i) p[i] = bf2f(f2bf(std::exp(s[i] - maximum) / total));
        float acc[kDim];
        for (int d = 0; d < kDim; ++d) acc[d] = 0.0f;
        for (int i = 0; i < n; ++i) {
            const uint16_t* v = value_row(key_start + i);
            for (int d = 0; d < kDim; ++d) acc[d] = std::fmaf(p[i], bf2f(v[d]), acc[d]);
        }
        for (int d = 0; d < kDim; ++d) out[d] = f2bf(acc[d]);
        return;
    }
    // ONLINE / FP32: fp32 probabilities, normalisation after the accumulation.
    float maximum = -INFINITY;
    for (int i = 0; i < n; ++i) maximum = maximum > s[i] ? maximum : s[i];
    float total = 0.0f;
    float acc[kDim];
    for (int d = 0; d < kDim; ++d) acc[d] = 0.0f;
    for (int i = 0; i < n; ++i) {
        const float p = std::exp(s[i] - maximum);
        total += p;
        const uint16_t* v = value_row(key_start + i);
        for (int d = 0; d < kDim; ++d) acc[d] = std::fmaf(p, bf2f(v[d]), acc[d]);
    }
    for (int d = 0; d < kDim; ++d) out[d] = f2bf(acc[d] / total);
}

// The predictor's topology for key_length <= 32: one wave per softmax row with lane =
// key, tree max / tree sum, and P.V as lane-strided fmaf + 32-lane tree
// (R17:12449-12574 == 9544-9601 + 9666-9697).  `masked_from` >= 0 marks keys that the
// staged causal mask replaced by bf16 -inf (R17:9516-9523).
void attend_predictor(const uint16_t* q, const RowPtr& key_row, const RowPtr& value_row,
                      int key_length, int masked_from, float scale, uint16_t* out) {
    float s[32];
    for (int l = 0; l < 32; ++l) s[l] = -INFINITY;
    for (int i = 0; i < key_length; ++i) {
        s[i] = score_from_dot(qk_dot(q, key_row(i)), scale, QMO_POLICY_REFERENCE);
        if (masked_from >= 0 && i >= masked_from) s[i] = bf2f(0xff80);
    }
    // max tree; the `lane + offset < 32` guard (R17:12463-12480) only changes lanes that
    // do not feed lane 0.
    const float maximum = wave32_max(s);
    float e[32];
    for (int l = 0; l < 32; ++l) e[l] = l < key_length ? std::exp(s[l] - maximum) : 0.0f;
    const float total = wave32_sum(e);
    float p[32];
    for (int l = 0; l < 32; ++l) p[l] = l < key_length ? bf2f(f2bf(e[l] / total)) : 0.0f;
    for (int d = 0; d < kDim; ++d) {
        float lanes[32];
        for (int l = 0; l < 32; ++l) {
            lanes[l] = 0.0f;
            if (l < key_length) lanes[l] = std::fmaf(p[l], bf2f(value_row(l)[d]), 0.0f);
        }
        out[d] = f2bf(wave32_sum(lanes));
    }
}

void parallel_for(int64_t n, int n_threads, const std::function<void(int64_t)>& body) {
    if (n_threads <= 1 || n <= 1) {
        for (int64_t i = 0; i < n; ++i) body(i);
        return;
    }
    const int workers = static_cast<int>(std::min<int64_t>(n_threads, n));
    std::vector<std::thread> pool;
    pool.reserve(workers);
    for (int w = 0; w < workers; ++w) {
        pool.emplace_back([&, w]() {
            for (int64_t i = w; i < n; i += workers) body(i);
        });
    }
    for (auto& t : pool) t.join();
}

inline uint64_t splitmix_at(uint64_t seed, uint64_t k) {
    // k-th output (k >= 1) of the SplitMix64 stream seeded with `seed`
    // (generator of R17:7108-7130: state += golden; mix(state)).
    uint64_t z = seed + k * 0x9e3779b97f4a7c15ULL;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
    return z ^ (z >> 31);
}

bool cache_ok(const qm_kv_cache* c) {
    return c && c->k_pool && c->v_pool && c->head_dim == kDim && c->stride_token == kDim
        && c->page_size > 0 && c->n_pages > 0 && c->kv_heads > 0;
}

}  // namespace

extern "C" {

// ---- scalar helpers ------------------------------------------------------------------
uint16_t qmo_f32_to_bf16(float v) { return f2bf(v); }
float qmo_bf16_to_f32(uint16_t v) { return bf2f(v); }

void qmo_f32_to_bf16_array(const float* in, uint16_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = f2bf(in[i]);
}
void qmo_bf16_to_f32_array(const uint16_t* in, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = bf2f(in[i]);
}

float qmo_head_sum_squares(const uint16_t* x) { return head_sum_squares(x); }

// ---- seeded synthetic inputs (owned by this repo; SplitMix64 -> Box-Muller) ----------
// Element i uses stream outputs 2i+1 and 2i+2, so the result does not depend on the
// thread count.
void qmo_fill_normal_bf16(uint16_t* out, int64_t n, uint64_t seed, float mean, float stdev,
                          int n_threads) {
    const int64_t chunk = 1 << 16;
    const int64_t chunks = (n + chunk - 1) / chunk;
    parallel_for(chunks, n_threads, [&](int64_t c) {
        const int64_t lo = c * chunk, hi = std::min(n, lo + chunk);
        for (int64_t i = lo; i < hi; ++i) {
            const uint64_t a = splitmix_at(seed, 2 * static_cast<uint64_t>(i) + 1);
            const uint64_t b = splitmix_at(seed, 2 * static_cast<uint64_t>(i) + 2);
            const double u1 = (static_cast<double>(a >> 11) + 1.0) * (1.0 / 9007199254740992.0);
            const double u2 = static_cast<double>(b >> 11) * (1.0 / 9007199254740992.0);
            const double z = std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586477 * u2);
            out[i] = f2bf(static_cast<float>(mean + stdev * z));
        }
    });
}

// Integers uniform in [lo, hi] (inclusive).
void qmo_fill_uniform_int(int32_t* out, int64_t n, uint64_t seed, int32_t lo, int32_t hi) {
    const uint64_t span = static_cast<uint64_t>(static_cast<int64_t>(hi) - lo + 1);
    for (int64_t i = 0; i < n; ++i) {
        out[i] = static_cast<int32_t>(lo + static_cast<int64_t>(
            splitmix_at(seed, static_cast<uint64_t>(i) + 1) % span));
    }
}

// Seeded Fisher-Yates permutation of 0..n-1.
void qmo_permutation(int32_t* out, int64_t n, uint64_t seed) {
    for (int64_t i = 0; i < n; ++i) out[i] = static_cast<int32_t>(i);
    for (int64_t i = n - 1; i > 0; --i) {
        const uint64_t j = splitmix_at(seed, static_cast<uint64_t>(n - i)) % static_cast<uint64_t>(i + 1);
        std::swap(out[i], out[j]);
    }
}

// ---- RoPE table: make_talker_rope R17:21576-21590, PersistentPredictor::make_rope
// R17:13161-13197 -------------------------------------------------------------------------
int32_t qmo_rope_table(int32_t rows, int32_t start, int32_t head_dim, double theta,
                       uint16_t* cos_out, uint16_t* sin_out) {
    if (rows < 0 || start < 0 || head_dim <= 0 || (head_dim & 1)) return QM_ERR_GEOMETRY;
    const int half = head_dim / 2;
    for (int row = 0; row < rows; ++row) {
        const double pos = static_cast<double>(start + row);
        for (int i = 0; i < half; ++i) {
            const double inv = std::pow(theta, -2.0 * static_cast<double>(i)
                                                   / static_cast<double>(head_dim));
            const double a = pos * inv;
            const uint16_t c = f2bf(static_cast<float>(std::cos(a)));
            const uint16_t s = f2bf(static_cast<float>(std::sin(a)));
            const size_t b = static_cast<size_t>(row) * head_dim;
            cos_out[b + i] = c;
            cos_out[b + i + half] = c;
            sin_out[b + i] = s;
            sin_out[b + i + half] = s;
        }
    }
    return QM_OK;
}

// ---- (1) fused norm + RoPE + append: R17:15365-15526 (talker), 12133-12307 (predictor) ---
int32_t qmo_qk_norm_rope_kv_append(
    const uint16_t* q, const uint16_t* k, const uint16_t* v,
    const uint16_t* q_norm_w, const uint16_t* k_norm_w,
    const uint16_t* cos_row, const uint16_t* sin_row,
    uint16_t* q_rotated,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    int32_t q_heads, int32_t cache_position, float epsilon) {
    if (!q || !k || !v || !q_norm_w || !k_norm_w || !cos_row || !sin_row || !q_rotated)
        return QM_ERR_NULL;
    if (!cache_ok(cache)) return QM_ERR_GEOMETRY;
    if (slot_offset(cache, page_table, max_pages, cache_position, 0) < 0)
        return QM_ERR_SLOT_RANGE;
    uint16_t tmp[kDim];
    for (int h = 0; h < q_heads; ++h) {
        head_rmsnorm(q + h * kDim, q_norm_w, epsilon, tmp);
        head_rope(tmp, cos_row, sin_row, q_rotated + h * kDim);
    }
    for (int h = 0; h < cache->kv_heads; ++h) {
        const int64_t off = slot_offset(cache, page_table, max_pages, cache_position, h);
        head_rmsnorm(k + h * kDim, k_norm_w, epsilon, tmp);
        head_rope(tmp, cos_row, sin_row, cache->k_pool + off);
        // V is appended un-normalised and un-rotated (R17:15515-15524).
        std::memcpy(cache->v_pool + off, v + h * kDim, kDim * sizeof(uint16_t));
    }
    return QM_OK;
}

int32_t qmo_qk_norm_rope_kv_append_ragged(
    const uint16_t* q, const uint16_t* k, const uint16_t* v,
    const uint16_t* q_norm_w, const uint16_t* k_norm_w,
    const uint16_t* cos_rows, const uint16_t* sin_rows, int32_t rope_by_position,
    uint16_t* q_rotated,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    const int32_t* positions, int32_t n_streams,
    int32_t q_heads, float epsilon, uint32_t* status) {
    if (!positions || !page_table) return QM_ERR_NULL;
    if (!cache_ok(cache)) return QM_ERR_GEOMETRY;
    for (int s = 0; s < n_streams; ++s) {
        const int32_t pos = positions[s];
        const int32_t* pt = page_table + static_cast<int64_t>(s) * max_pages;
        if (pos < 0 || pos / cache->page_size >= max_pages) {
            if (status) *status |= QM_STATUS_BAD_POSITION;
            continue;
        }
        if (slot_offset(cache, pt, max_pages, pos, 0) < 0) {
            if (status) *status |= QM_STATUS_BAD_PAGE;
            continue;
        }
        const int64_t row = rope_by_position ? pos : s;
        const int32_t rc = qmo_qk_norm_rope_kv_append(
            q + static_cast<int64_t>(s) * q_heads * kDim,
            k + static_cast<int64_t>(s) * cache->kv_heads * kDim,
            v + static_cast<int64_t>(s) * cache->kv_heads * kDim,
            q_norm_w, k_norm_w, cos_rows + row * kDim, sin_rows + row * kDim,
            q_rotated + static_cast<int64_t>(s) * q_heads * kDim,
            cache, pt, max_pages, q_heads, pos, epsilon);
        if (rc != QM_OK) return rc;
    }
    return QM_OK;
}

// ---- prefill front half: rmsnorm_kernel rows = S*heads, dim 128 (R17:8276-8338) followed by
// talker_rope_rows_kernel (R17:15531-15625) -------------------------------------------------
int32_t qmo_norm_rope_rows(const uint16_t* in, const uint16_t* norm_w,
                           const uint16_t* cos_rows, const uint16_t* sin_rows,
                           uint16_t* out, int32_t rows, int32_t heads, float epsilon) {
    if (!in || !cos_rows || !sin_rows || !out) return QM_ERR_NULL;
    if (rows < 0 || heads <= 0) return QM_ERR_ARGUMENT;
    uint16_t tmp[kDim];
    for (int64_t r = 0; r < rows; ++r) {
        for (int h = 0; h < heads; ++h) {
            const uint16_t* x = in + (r * heads + h) * kDim;
            if (norm_w) {
                head_rmsnorm(x, norm_w, epsilon, tmp);
                x = tmp;
            }
            head_rope(x, cos_rows + r * kDim, sin_rows + r * kDim, out + (r * heads + h) * kDim);
        }
    }
    return QM_OK;
}

// scatter_prefill_kv (R17:15630-15687) / scatter_decode_kv (R17:15701-15740)
int32_t qmo_scatter_kv(const uint16_t* key, const uint16_t* value,
                       const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
                       int32_t rows, int32_t first_position) {
    if (!key || !value) return QM_ERR_NULL;
    if (!cache_ok(cache)) return QM_ERR_GEOMETRY;
    if (rows < 0 || first_position < 0) return QM_ERR_ARGUMENT;
    for (int64_t r = 0; r < rows; ++r) {
        if (slot_offset(cache, page_table, max_pages, first_position + r, 0) < 0)
            return QM_ERR_SLOT_RANGE;
    }
    for (int64_t r = 0; r < rows; ++r) {
        for (int h = 0; h < cache->kv_heads; ++h) {
            const int64_t off = slot_offset(cache, page_table, max_pages, first_position + r, h);
            const int64_t src = (r * cache->kv_heads + h) * kDim;
            std::memcpy(cache->k_pool + off, key + src, kDim * sizeof(uint16_t));
            std::memcpy(cache->v_pool + off, value + src, kDim * sizeof(uint16_t));
        }
    }
    return QM_OK;
}

// ---- attention over a (paged) cache: talker_attention_kernel R17:15744-16006, with
// query_length == 1 identical to talker_attention_gqa2_m1_locality_kernel R17:16014-16203 ---
// query, out [query_length][q_heads][128]; row i attends keys [key_start, cache_before+i+1).
int32_t qmo_attention(
    const uint16_t* query,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    uint16_t* out,
    int32_t query_length, int32_t cache_before, int32_t q_heads,
    int32_t sliding_window, float scale, int32_t policy, int32_t n_threads) {
    if (!query || !out) return QM_ERR_NULL;
    if (!cache_ok(cache) || q_heads <= 0 || q_heads % cache->kv_heads) return QM_ERR_GEOMETRY;
    if (query_length < 0 || cache_before < 0) return QM_ERR_ARGUMENT;
    if (query_length > 0
        && slot_offset(cache, page_table, max_pages, cache_before + query_length - 1, 0) < 0)
        return QM_ERR_SLOT_RANGE;
    const int group = q_heads / cache->kv_heads;
    parallel_for(static_cast<int64_t>(query_length) * q_heads, n_threads, [&](int64_t item) {
        const int qi = static_cast<int>(item / q_heads);
        const int qh = static_cast<int>(item % q_heads);
        const int kvh = qh / group;                       // R17:15780-15782
        const int key_end = cache_before + qi + 1;        // R17:15784-15789
        const int window_start = key_end - sliding_window;
        const int key_start = sliding_window > 0 ? (window_start > 0 ? window_start : 0) : 0;
        RowPtr krow = [&](int t) {
            return cache->k_pool + slot_offset(cache, page_table, max_pages, t, kvh);
        };
        RowPtr vrow = [&](int t) {
            return cache->v_pool + slot_offset(cache, page_table, max_pages, t, kvh);
        };
        const int64_t base = (static_cast<int64_t>(qi) * q_heads + qh) * kDim;
        attend_talker(query + base, krow, vrow, key_start, key_end, scale, policy, out + base);
    });
    return QM_OK;
}

// Ragged multi-stream decode = qmo_attention(query_length 1) per stream.
int32_t qmo_decode_attention_ragged(
    const uint16_t* query,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    const int32_t* seq_lens, int32_t n_streams,
    uint16_t* out, int32_t q_heads, float scale, int32_t policy, int32_t n_threads) {
    if (!query || !out || !seq_lens || !page_table) return QM_ERR_NULL;
    if (!cache_ok(cache) || q_heads <= 0 || q_heads % cache->kv_heads) return QM_ERR_GEOMETRY;
    int32_t rc_all = QM_OK;
    parallel_for(n_streams, n_threads, [&](int64_t s) {
        const int64_t base = s * q_heads * kDim;
        if (seq_lens[s] <= 0) {
            std::memset(out + base, 0, sizeof(uint16_t) * q_heads * kDim);
            return;
        }
        const int32_t rc = qmo_attention(query + base, cache, page_table + s * max_pages,
                                         max_pages, out + base, 1, seq_lens[s] - 1, q_heads,
                                         -1, scale, policy, 1);
        if (rc != QM_OK) rc_all = rc;
    });
    return rc_all;
}

// ---- causal prefill over contiguous K/V (+ paged write): talker_attention_kernel with
// cache_before == 0 after scatter_prefill_cache (R17:16703-16717) --------------------------
int32_t qmo_prefill_attention_causal(
    const uint16_t* query, const uint16_t* key, const uint16_t* value, uint16_t* out,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    int32_t batch, int32_t seq, int32_t q_heads, int32_t kv_heads, float scale,
    int32_t policy, int32_t n_threads) {
    if (!query || !key || !value || !out) return QM_ERR_NULL;
    if (q_heads <= 0 || kv_heads <= 0 || q_heads % kv_heads) return QM_ERR_GEOMETRY;
    if (batch < 0 || seq < 0) return QM_ERR_ARGUMENT;
    if (cache) {
        if (!cache_ok(cache) || cache->kv_heads != kv_heads) return QM_ERR_GEOMETRY;
        for (int b = 0; b < batch; ++b) {
            const int32_t rc = qmo_scatter_kv(
                key + static_cast<int64_t>(b) * seq * kv_heads * kDim,
                value + static_cast<int64_t>(b) * seq * kv_heads * kDim, cache,
                page_table ? page_table + static_cast<int64_t>(b) * max_pages : nullptr,
                max_pages, seq, 0);
            if (rc != QM_OK) return rc;
        }
    }
    const int group = q_heads / kv_heads;
    parallel_for(static_cast<int64_t>(batch) * seq * q_heads, n_threads, [&](int64_t item) {
        const int qh = static_cast<int>(item % q_heads);
        const int64_t t = item / q_heads;
        const int qi = static_cast<int>(t % seq);
        const int b = static_cast<int>(t / seq);
        const int kvh = qh / group;
        const uint16_t* kb = key + static_cast<int64_t>(b) * seq * kv_heads * kDim;
        const uint16_t* vb = value + static_cast<int64_t>(b) * seq * kv_heads * kDim;
        RowPtr krow = [&](int i) { return kb + (static_cast<int64_t>(i) * kv_heads + kvh) * kDim; };
        RowPtr vrow = [&](int i) { return vb + (static_cast<int64_t>(i) * kv_heads + kvh) * kDim; };
        const int64_t base = ((static_cast<int64_t>(b) * seq + qi) * q_heads + qh) * kDim;
        attend_talker(query + base, krow, vrow, 0, qi + 1, scale, policy, out + base);
    });
    return QM_OK;
}

// ---- predictor -------------------------------------------------------------------------
// predictor_attention_gqa2_m1_kernel R17:12314-12575 over a flat [8][16][128] cache.
int32_t qmo_predictor_attention_m1(const uint16_t* query, const uint16_t* key_cache,
                                   const uint16_t* value_cache, uint16_t* out,
                                   int32_t key_length) {
    if (!query || !key_cache || !value_cache || !out) return QM_ERR_NULL;
    if (key_length < 1 || key_length > 16) return QM_ERR_ARGUMENT;
    uint32_t sb = 0x3db504f3U;  // kAttentionScaleBits, R17:9354-9356
    float scale;
    std::memcpy(&scale, &sb, 4);
    for (int qh = 0; qh < 16; ++qh) {
        const int kvh = qh / 2;
        RowPtr krow = [&](int t) { return key_cache + (static_cast<int64_t>(kvh) * 16 + t) * kDim; };
        RowPtr vrow = [&](int t) { return value_cache + (static_cast<int64_t>(kvh) * 16 + t) * kDim; };
        attend_predictor(query + qh * kDim, krow, vrow, key_length, -1, scale, out + qh * kDim);
    }
    return QM_OK;
}

// The staged six-kernel attention of step 0 (R17:9369-9745, dispatch 13300-13386):
// query in BHSD [16][rows][128], cache [8][16][128], causal mask over key_length keys,
// output transposed to [rows][16][128].
int32_t qmo_predictor_attention_staged(const uint16_t* query_bhsd, const uint16_t* key_cache,
                                       const uint16_t* value_cache, uint16_t* out_bshd,
                                       int32_t rows, int32_t key_length, int32_t causal) {
    if (!query_bhsd || !key_cache || !value_cache || !out_bshd) return QM_ERR_NULL;
    if (rows < 1 || key_length < 1 || key_length > 16) return QM_ERR_ARGUMENT;
    uint32_t sb = 0x3db504f3U;
    float scale;
    std::memcpy(&scale, &sb, 4);
    for (int qh = 0; qh < 16; ++qh) {
        const int kvh = qh / 2;
        RowPtr krow = [&](int t) { return key_cache + (static_cast<int64_t>(kvh) * 16 + t) * kDim; };
        RowPtr vrow = [&](int t) { return value_cache + (static_cast<int64_t>(kvh) * 16 + t) * kDim; };
        for (int r = 0; r < rows; ++r) {
            const int masked_from = causal ? r + 1 : -1;  // key_index > query_index (R17:9517-9520)
            attend_predictor(query_bhsd + (static_cast<int64_t>(qh) * rows + r) * kDim, krow, vrow,
                             key_length, masked_from < key_length ? masked_from : -1, scale,
                             out_bshd + (static_cast<int64_t>(r) * 16 + qh) * kDim);
        }
    }
    return QM_OK;
}

// The three layout kernels in front of the staged attention of step 0 (call site R17:13663-13699).
// transpose_bshd_to_bhsd_kernel R17:8366-8400: [rows][heads][128] -> [heads][rows][128].
int32_t qmo_predictor_transpose(const uint16_t* input, uint16_t* output, int32_t rows, int32_t heads) {
    if (!input || !output) return QM_ERR_NULL;
    if (rows < 0 || heads <= 0) return QM_ERR_ARGUMENT;
    const int64_t count = static_cast<int64_t>(rows) * heads * kDim;
    for (int64_t index = 0; index < count; ++index) {
        const int d = static_cast<int>(index % kDim);
        const int64_t t = index / kDim;
        const int64_t head = t % heads;
        const int64_t sequence = t / heads;
        output[(head * rows + sequence) * kDim + d] = input[index];
    }
    return QM_OK;
}

// apply_rope_kernel R17:8403-8488 on a BHSD tensor [heads][rows][128]: element index ->
// sequence = (index / 128) % rows, head = (index / 128) / rows; cos/sin row = sequence;
// bf16(bf16(x * cos) + bf16(+-x[d +- 64] * sin)), the sign negative for d < 64.
int32_t qmo_predictor_rope_bhsd(const uint16_t* input, const uint16_t* cosine, const uint16_t* sine,
                                uint16_t* output, int32_t rows, int32_t heads) {
    if (!input || !cosine || !sine || !output) return QM_ERR_NULL;
    if (rows < 0 || heads <= 0) return QM_ERR_ARGUMENT;
    const int64_t count = static_cast<int64_t>(rows) * heads * kDim;
    for (int64_t index = 0; index < count; ++index) {
        const int d = static_cast<int>(index % kDim);
        const int64_t t = index / kDim;
        const int64_t sequence = t % rows;
        const int64_t head = t / rows;
        const int rd = d < kDim / 2 ? d + kDim / 2 : d - kDim / 2;
        const float sign = d < kDim / 2 ? -1.0f : 1.0f;
        const int64_t base = (head * rows + sequence) * kDim;
        const float value = bf2f(input[base + d]);
        const float rotated = sign * bf2f(input[base + rd]);
        const uint16_t first = f2bf(value * bf2f(cosine[sequence * kDim + d]));
        const uint16_t second = f2bf(rotated * bf2f(sine[sequence * kDim + d]));
        output[index] = f2bf(bf2f(first) + bf2f(second));
    }
    return QM_OK;
}

// update_cache_kernel R17:8491-8529: source [8][rows][128] (BHSD) -> cache [8][16][128] at
// positions start .. start + rows - 1 of every head.  The reference has no range guard; here a
// run past the 16 positions is an error and nothing is written.
int32_t qmo_predictor_update_cache(const uint16_t* source, uint16_t* cache, int32_t rows, int32_t start) {
    if (!source || !cache) return QM_ERR_NULL;
    if (rows < 0 || start < 0) return QM_ERR_ARGUMENT;
    if (start + rows > 16) return QM_ERR_SLOT_RANGE;
    const int64_t count = static_cast<int64_t>(8) * rows * kDim;
    for (int64_t index = 0; index < count; ++index) {
        const int d = static_cast<int>(index % kDim);
        const int64_t t = index / kDim;
        const int64_t sequence = t % rows;
        const int64_t head = t / rows;
        cache[(head * 16 + start + sequence) * kDim + d] = source[index];
    }
    return QM_OK;
}

// The whole step loop of one (frame, layer) unit after another, schedule of
// PersistentPredictor::capture_step R17:13592-13596: row r is appended at position r and
// attends keys 0..r.
int32_t qmo_predictor_attention_loop(
    const uint16_t* q, const uint16_t* k, const uint16_t* v,
    const uint16_t* q_norm_w, const uint16_t* k_norm_w,
    const uint16_t* cos_rows, const uint16_t* sin_rows,
    uint16_t* context_out, uint16_t* k_cache_out, uint16_t* v_cache_out,
    int32_t units, int32_t n_layers, int32_t rows, int32_t first_rows,
    float epsilon, int32_t n_threads) {
    if (!q || !k || !v || !q_norm_w || !k_norm_w || !cos_rows || !sin_rows || !context_out)
        return QM_ERR_NULL;
    if (units < 0 || n_layers <= 0 || rows < 1 || rows > 16) return QM_ERR_ARGUMENT;
    if (first_rows != 1 && first_rows != 2) return QM_ERR_ARGUMENT;
    if (first_rows > rows) return QM_ERR_ARGUMENT;
    parallel_for(units, n_threads, [&](int64_t u) {
        std::vector<uint16_t> kc(8 * 16 * kDim, 0), vc(8 * 16 * kDim, 0), qrot(16 * kDim);
        qm_kv_cache cache;
        cache.k_pool = kc.data();
        cache.v_pool = vc.data();
        cache.stride_page = 0;
        cache.stride_head = 16 * kDim;
        cache.stride_token = kDim;
        cache.page_size = 16;
        cache.n_pages = 1;
        cache.kv_heads = 8;
        cache.head_dim = kDim;
        const int layer = static_cast<int>(u % n_layers);
        for (int r = 0; r < rows; ++r) {
            const int64_t row = u * rows + r;
            qmo_qk_norm_rope_kv_append(
                q + row * 16 * kDim, k + row * 8 * kDim, v + row * 8 * kDim,
                q_norm_w + layer * kDim, k_norm_w + layer * kDim,
                cos_rows + r * kDim, sin_rows + r * kDim, qrot.data(),
                &cache, nullptr, 1, 16, r, epsilon);
            qmo_predictor_attention_m1(qrot.data(), kc.data(), vc.data(),
                                       context_out + row * 16 * kDim, r + 1);
        }
        if (k_cache_out) std::memcpy(k_cache_out + u * 8 * 16 * kDim, kc.data(), kc.size() * 2);
        if (v_cache_out) std::memcpy(v_cache_out + u * 8 * 16 * kDim, vc.data(), vc.size() * 2);
    });
    return QM_OK;
}

// ---- M = 1 weight-streaming linears ------------------------------------------------------------------
// One output scalar as one 32-lane wave of talker_linear_fused_kernel / talker_qkv_fused_kernel
// computes it (R17:15239-15266, 15340-15360): lane l accumulates k = l, l+32, ... with fmaf in
// increasing k, the 32 lane sums go through the shuffle tree, lane 0 adds the bias in fp32 and
// rounds to bf16; with a residual the stored value is bf16(residual + bf16(result)).
static uint16_t linear_m1_scalar(const uint16_t* input, const uint16_t* weight_row, const uint16_t* bias,
                                 const uint16_t* residual, int out, int reduction_columns) {
    float lanes[32];
    for (int l = 0; l < 32; ++l) {
        float acc = 0.0f;
        for (int k = l; k < reduction_columns; k += 32) acc = std::fmaf(bf2f(input[k]), bf2f(weight_row[k]), acc);
        lanes[l] = acc;
    }
    float a = wave32_sum(lanes);
    if (bias) a += bf2f(bias[out]);
    const uint16_t v = f2bf(a);
    return residual ? f2bf(bf2f(residual[out]) + bf2f(v)) : v;
}

// talker_linear_fused_kernel + launch_linear_m1 (R17:15201-15268, 17473-17511): weight is
// [output_columns][reduction_columns] row-major; bias and residual may be NULL.
int32_t qmo_linear_m1(const uint16_t* input, const uint16_t* weight, const uint16_t* bias,
                      const uint16_t* residual, uint16_t* output, int32_t output_columns,
                      int32_t reduction_columns, int32_t n_threads) {
    if (!input || !weight || !output) return QM_ERR_NULL;
    if (output_columns < 0 || reduction_columns < 0) return QM_ERR_ARGUMENT;
    parallel_for(output_columns, n_threads, [&](int64_t o) {
        output[o] = linear_m1_scalar(input, weight + o * reduction_columns, bias, residual,
                                     static_cast<int>(o), reduction_columns);
    });
    return QM_OK;
}

// talker_qkv_fused_kernel + launch_qkv_m1 (R17:15272-15362, 17513-17567): three linears over one
// staged input; output row r of the concatenation q | k | v reads its own weight, bias and output.
int32_t qmo_qkv_m1(const uint16_t* input, const uint16_t* q_weight, const uint16_t* q_bias,
                   const uint16_t* k_weight, const uint16_t* k_bias, const uint16_t* v_weight,
                   const uint16_t* v_bias, uint16_t* q_output, uint16_t* k_output, uint16_t* v_output,
                   int32_t hidden, int32_t q_dim, int32_t kv_dim, int32_t n_threads) {
    if (!input || !q_weight || !k_weight || !v_weight || !q_output || !k_output || !v_output) return QM_ERR_NULL;
    if (hidden < 0 || q_dim < 0 || kv_dim < 0) return QM_ERR_ARGUMENT;
    parallel_for(static_cast<int64_t>(q_dim) + 2 * kv_dim, n_threads, [&](int64_t first) {
        if (first < q_dim) {
            q_output[first] = linear_m1_scalar(input, q_weight + first * hidden, q_bias, nullptr,
                                               static_cast<int>(first), hidden);
        } else if (first < q_dim + kv_dim) {
            const int64_t r = first - q_dim;
            k_output[r] = linear_m1_scalar(input, k_weight + r * hidden, k_bias, nullptr, static_cast<int>(r), hidden);
        } else {
            const int64_t r = first - q_dim - kv_dim;
            v_output[r] = linear_m1_scalar(input, v_weight + r * hidden, v_bias, nullptr, static_cast<int>(r), hidden);
        }
    });
    return QM_OK;
}

// Sum over a 256-thread block of per-thread partial sums, thread t having accumulated the
// columns t, t+256, ... with fmaf (R17:8291-8301, 16221-16251), reduced by block_reduce_sum /
// talker_block_sum (eight 32-lane trees, then a tree over the eight results).
static float strided_sum_squares_256(const uint16_t* x, int dimension) {
    float per_thread[256];
    for (int t = 0; t < 256; ++t) {
        float acc = 0.0f;
        for (int c = t; c < dimension; c += 256) {
            const float v = bf2f(x[c]);
            acc = std::fmaf(v, v, acc);
        }
        per_thread[t] = acc;
    }
    return block_sum(per_thread, 256);
}

// rmsnorm_kernel + launch_rmsnorm (R17:8276-8338, 8908-8929; 256 threads per row, epsilon
// kRmsEpsilon = 1e-6 passed in): out = bf16(bf16(x * inverse_rms) * weight).
int32_t qmo_rmsnorm_rows(const uint16_t* input, const uint16_t* weight, uint16_t* output, int32_t rows,
                         int32_t dimension, float epsilon, int32_t n_threads) {
    if (!input || !weight || !output) return QM_ERR_NULL;
    if (rows < 0 || dimension <= 0) return QM_ERR_ARGUMENT;
    parallel_for(rows, n_threads, [&](int64_t r) {
        const uint16_t* x = input + r * dimension;
        const float sum = strided_sum_squares_256(x, dimension);
        const float inv = 1.0f / std::sqrt(sum / static_cast<float>(dimension) + epsilon);
        for (int c = 0; c < dimension; ++c) {
            const uint16_t n = f2bf(bf2f(x[c]) * inv);
            output[r * dimension + c] = f2bf(bf2f(n) * bf2f(weight[c]));
        }
    });
    return QM_OK;
}

// talker_add_postnorm_fused_kernel + launch_add_postnorm_m1 (R17:16205-16286, 17817-17846):
// residual = bf16(hidden + attention); normalized = bf16(bf16(residual * inverse_rms) * weight),
// the statistic taken over the rounded residual.
int32_t qmo_add_postnorm_m1(const uint16_t* hidden, const uint16_t* attention, const uint16_t* norm_weight,
                            uint16_t* residual, uint16_t* normalized, int32_t dimension, float epsilon) {
    if (!hidden || !attention || !norm_weight || !residual || !normalized) return QM_ERR_NULL;
    if (dimension <= 0) return QM_ERR_ARGUMENT;
    for (int c = 0; c < dimension; ++c) residual[c] = f2bf(bf2f(hidden[c]) + bf2f(attention[c]));
    const float sum = strided_sum_squares_256(residual, dimension);
    const float inv = 1.0f / std::sqrt(sum / static_cast<float>(dimension) + epsilon);
    for (int c = 0; c < dimension; ++c) {
        const uint16_t n = f2bf(bf2f(residual[c]) * inv);
        normalized[c] = f2bf(bf2f(n) * bf2f(norm_weight[c]));
    }
    return QM_OK;
}

// talker_gate_up_swiglu_fused_kernel + launch_gate_up_swiglu_m1 (R17:16289-16362, 17848-17890):
// per channel two dot products in the M = 1 linear's order (no bias), each rounded to bf16;
// act = bf16(g / (1 + expf(-g))); out = bf16(act * u).
int32_t qmo_gate_up_swiglu_m1(const uint16_t* input, const uint16_t* gate_weight, const uint16_t* up_weight,
                              uint16_t* output, int32_t hidden, int32_t intermediate, int32_t n_threads) {
    if (!input || !gate_weight || !up_weight || !output) return QM_ERR_NULL;
    if (hidden < 0 || intermediate < 0) return QM_ERR_ARGUMENT;
    parallel_for(intermediate, n_threads, [&](int64_t ch) {
        const uint16_t gb = linear_m1_scalar(input, gate_weight + ch * hidden, nullptr, nullptr, 0, hidden);
        const uint16_t ub = linear_m1_scalar(input, up_weight + ch * hidden, nullptr, nullptr, 0, hidden);
        const float gv = bf2f(gb);
        const uint16_t act = f2bf(gv / (1.0f + std::exp(-gv)));
        output[ch] = f2bf(bf2f(act) * bf2f(ub));
    });
    return QM_OK;
}

// ---- the code predictor's M = 1 linears ------------------------------------------------------------
// predictor_linear_m1_fused_kernel, predictor_qkv_m1_fused_kernel and
// predictor_gate_up_swiglu_m1_kernel (R17:12579-12654, 12046-12130, 12736-12815) walk a row in
// another order than the talker's: lane l takes the element pairs k = 2l, 2l + 64, ... (loop
// condition k + 1 < columns) and adds x[k] w[k] and then x[k+1] w[k+1] to its accumulator
// (predictor_bf16_dot2_accumulate, R17:8193-8230, in its portable form: two fmaf; the gfx1100 build
// uses that chip's dot2 instruction instead, whose rounding is the hardware's and is not restated
// here); a last odd column is added by lane 0 after its pairs; the same shuffle tree; no bias.
static uint16_t predictor_linear_m1_scalar(const uint16_t* input, const uint16_t* weight_row,
                                           const uint16_t* residual, int out, int reduction_columns) {
    float lanes[32];
    for (int l = 0; l < 32; ++l) {
        float acc = 0.0f;
        for (int k = 2 * l; k + 1 < reduction_columns; k += 64) {
            acc = std::fmaf(bf2f(input[k]), bf2f(weight_row[k]), acc);
            acc = std::fmaf(bf2f(input[k + 1]), bf2f(weight_row[k + 1]), acc);
        }
        lanes[l] = acc;
    }
    if (reduction_columns & 1) {
        const int k = reduction_columns - 1;
        lanes[0] = std::fmaf(bf2f(input[k]), bf2f(weight_row[k]), lanes[0]);
    }
    const uint16_t v = f2bf(wave32_sum(lanes));
    return residual ? f2bf(bf2f(residual[out]) + bf2f(v)) : v;
}

int32_t qmo_predictor_linear_m1(const uint16_t* input, const uint16_t* weight, const uint16_t* residual,
                                uint16_t* output, int32_t output_columns, int32_t reduction_columns,
                                int32_t n_threads) {
    if (!input || !weight || !output) return QM_ERR_NULL;
    if (output_columns < 0 || reduction_columns < 0) return QM_ERR_ARGUMENT;
    parallel_for(output_columns, n_threads, [&](int64_t o) {
        output[o] = predictor_linear_m1_scalar(input, weight + o * reduction_columns, residual,
                                               static_cast<int>(o), reduction_columns);
    });
    return QM_OK;
}

int32_t qmo_predictor_qkv_m1(const uint16_t* input, const uint16_t* q_weight, const uint16_t* k_weight,
                             const uint16_t* v_weight, uint16_t* q_output, uint16_t* k_output,
                             uint16_t* v_output, int32_t hidden, int32_t q_dim, int32_t kv_dim,
                             int32_t n_threads) {
    if (!input || !q_weight || !k_weight || !v_weight || !q_output || !k_output || !v_output) return QM_ERR_NULL;
    if (hidden < 0 || q_dim < 0 || kv_dim < 0) return QM_ERR_ARGUMENT;
    parallel_for(static_cast<int64_t>(q_dim) + 2 * kv_dim, n_threads, [&](int64_t first) {
        if (first < q_dim) {
            q_output[first] = predictor_linear_m1_scalar(input, q_weight + first * hidden, nullptr, 0, hidden);
        } else if (first < q_dim + kv_dim) {
            const int64_t r = first - q_dim;
            k_output[r] = predictor_linear_m1_scalar(input, k_weight + r * hidden, nullptr, 0, hidden);
        } else {
            const int64_t r = first - q_dim - kv_dim;
            v_output[r] = predictor_linear_m1_scalar(input, v_weight + r * hidden, nullptr, 0, hidden);
        }
    });
    return QM_OK;
}

int32_t qmo_predictor_gate_up_swiglu_m1(const uint16_t* input, const uint16_t* gate_weight,
                                        const uint16_t* up_weight, uint16_t* output, int32_t hidden,
                                        int32_t intermediate, int32_t n_threads) {
    if (!input || !gate_weight || !up_weight || !output) return QM_ERR_NULL;
    if (hidden < 0 || intermediate < 0) return QM_ERR_ARGUMENT;
    parallel_for(intermediate, n_threads, [&](int64_t ch) {
        const uint16_t gb = predictor_linear_m1_scalar(input, gate_weight + ch * hidden, nullptr, 0, hidden);
        const uint16_t ub = predictor_linear_m1_scalar(input, up_weight + ch * hidden, nullptr, 0, hidden);
        const float gv = bf2f(gb);
        const uint16_t act = f2bf(gv / (1.0f + std::exp(-gv)));
        output[ch] = f2bf(bf2f(act) * bf2f(ub));
    });
    return QM_OK;
}

// ---- final head: score processing, top-k sampler, history ---------------------------------------------
// SplitMix64 and the uniform draw of the sampler (R17:7353-7371).
static uint64_t splitmix64_next(uint64_t* state) {
    uint64_t z = *state + 0x9e3779b97f4a7c15ULL;
    *state = z;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
    return z ^ (z >> 31);
}

int32_t qmo_splitmix64(uint64_t* state, int32_t count, uint64_t* raw_out, double* uniform_out) {
    if (!state) return QM_ERR_NULL;
    for (int i = 0; i < count; ++i) {
        const uint64_t z = splitmix64_next(state);
        if (raw_out) raw_out[i] = z;
        if (uniform_out) uniform_out[i] = static_cast<double>(z >> 11) * (1.0 / 9007199254740992.0);
    }
    return QM_OK;
}

// gpu_sample_topk_f32_kernel / gpu_sample_topk_bf16_kernel (R17:7407-7518): all scores sorted by
// (score descending, id ascending) (gpu_sampler_better, R17:7347-7351 — a total order for
// scores without NaN, so the sorting network's result is the sorted sequence); over the first
// keep = min(top_k, vocab): maximum = score[0] / T, total = sum of exp(score / T - maximum) in
// double in that order; without a positive total the first id is returned and no number is
// drawn; else target = uniform * total and the first index whose running sum exceeds it.
static int32_t sample_sorted(const float* scores, int vocab, int top_k, float temperature, uint64_t* rng_state) {
    std::vector<int> order(vocab);
    for (int i = 0; i < vocab; ++i) order[i] = i;
    std::sort(order.begin(), order.end(), [&](int a, int b) {
        return scores[a] > scores[b] || (scores[a] == scores[b] && a < b);
    });
    const int keep = top_k < vocab ? top_k : vocab;
    const double inv_t = 1.0 / static_cast<double>(temperature);
    const double maximum = static_cast<double>(scores[order[0]]) * inv_t;
    double total = 0.0;
    for (int i = 0; i < keep; ++i) total += std::exp(static_cast<double>(scores[order[i]]) * inv_t - maximum);
    if (!(total > 0.0)) return order[0];
    const double uniform = static_cast<double>(splitmix64_next(rng_state) >> 11) * (1.0 / 9007199254740992.0);
    const double target = uniform * total;
    double cumulative = 0.0;
    for (int i = 0; i < keep; ++i) {
        cumulative += std::exp(static_cast<double>(scores[order[i]]) * inv_t - maximum);
        if (target < cumulative) return order[i];
    }
    return order[keep - 1];
}

// logits: float (is_bf16 == 0) or bf16 bit patterns, read from element `offset` on
// (last_row_offset of the bf16 kernel).  top_k <= 0 selects the arg-max kernels
// (argmax_final_head R17:14099-14143, argmax_bf16_kernel: highest score, lowest id among equals).
int32_t qmo_sample_topk(const void* logits, int32_t is_bf16, int32_t offset, int32_t vocab, int32_t top_k,
                        float temperature, uint64_t* rng_state, int32_t* output_id) {
    if (!logits || !output_id) return QM_ERR_NULL;
    if (vocab <= 0 || offset < 0) return QM_ERR_ARGUMENT;
    std::vector<float> scores(vocab);
    for (int i = 0; i < vocab; ++i)
        scores[i] = is_bf16 ? bf2f(static_cast<const uint16_t*>(logits)[offset + i])
                            : static_cast<const float*>(logits)[offset + i];
    if (top_k <= 0) {
        int best = 0;
        for (int i = 1; i < vocab; ++i)
            if (scores[i] > scores[best]) best = i;
        *output_id = best;
        return QM_OK;
    }
    if (!rng_state) return QM_ERR_NULL;
    *output_id = sample_sorted(scores.data(), vocab, top_k, temperature, rng_state);
    return QM_OK;
}

// cast_final_head_logits, repetition_penalty, suppress_tokens (R17:14025-14097), in that order:
// score = f32(logit); a token found in history[0 .. history_count) is multiplied by the penalty
// if negative, else by float(1) / float(penalty) (for 1.05: the constant 0x3f73cf3e, R17:14062);
// the end-of-sequence token is -inf while generation_index < 2; the last `suppressed_tail`
// tokens other than it are always -inf.
int32_t qmo_final_head_process(const uint16_t* logits, const int32_t* history, int32_t history_count,
                               int32_t generation_index, int32_t vocab, int32_t eos, int32_t suppressed_tail,
                               float penalty, float* scores) {
    if (!logits || !scores || (history_count > 0 && !history)) return QM_ERR_NULL;
    if (vocab <= 0 || history_count < 0) return QM_ERR_ARGUMENT;
    const float reciprocal = 1.0f / penalty;
    for (int token = 0; token < vocab; ++token) {
        float score = bf2f(logits[token]);
        bool repeated = false;
        for (int i = 0; i < history_count && !repeated; ++i) repeated = history[i] == token;
        if (repeated) score = score < 0.0f ? score * penalty : score * reciprocal;
        if (token == eos && generation_index < 2) score = -INFINITY;
        if (token >= vocab - suppressed_tail && token != eos) score = -INFINITY;
        scores[token] = score;
    }
    return QM_OK;
}

// The device side of NativeFinalHead::run_fast_device after the head projection
// (R17:14456-14545): process, sample (or arg-max when top_k <= 0), append the code to the history.
int32_t qmo_final_head_sample(const uint16_t* logits, int32_t* history, int32_t generation_index, int32_t vocab,
                              int32_t eos, int32_t suppressed_tail, float penalty, int32_t top_k,
                              float temperature, uint64_t* rng_state, int32_t* code_out, float* scores_out) {
    if (!logits || !history || !code_out) return QM_ERR_NULL;
    if (generation_index < 0) return QM_ERR_ARGUMENT;
    std::vector<float> scores(vocab > 0 ? vocab : 1);
    int32_t rc = qmo_final_head_process(logits, history, generation_index, generation_index, vocab, eos,
                                        suppressed_tail, penalty, scores.data());
    if (rc != QM_OK) return rc;
    if (scores_out) std::memcpy(scores_out, scores.data(), sizeof(float) * vocab);
    rc = qmo_sample_topk(scores.data(), 0, 0, vocab, top_k, temperature, rng_state, code_out);
    if (rc != QM_OK) return rc;
    history[generation_index] = *code_out;
    return QM_OK;
}

// ---- linears over token rows (the prompt pass) -----------------------------------------------------------
// native_ops::linear_wave32_bf16_f32acc_kernel (R17:126-196; NativeTalkerEngine::linear_generic
// :17453-17472): every (row, column) is the M = 1 linear's scalar — same chains, tree, bias.
// `residual` folds add_bf16_kernel (R17:8729-8744) behind it; the gate/up form folds swiglu_kernel
// (R17:8745-8770) behind two such linears: exactly the M = 1 SwiGLU arithmetic, row by row.
int32_t qmo_linear_rows(const uint16_t* input, const uint16_t* weight, const uint16_t* bias,
                        const uint16_t* residual, uint16_t* output, int32_t rows, int32_t output_columns,
                        int32_t reduction_columns, int32_t n_threads) {
    if (!input || !weight || !output) return QM_ERR_NULL;
    if (rows < 0 || output_columns < 0 || reduction_columns < 0) return QM_ERR_ARGUMENT;
    parallel_for(static_cast<int64_t>(rows) * output_columns, n_threads, [&](int64_t at) {
        const int64_t r = at / output_columns;
        const int o = static_cast<int>(at % output_columns);
        output[at] = linear_m1_scalar(input + r * reduction_columns, weight + static_cast<int64_t>(o) * reduction_columns,
                                      bias, residual ? residual + r * output_columns : nullptr, o, reduction_columns);
    });
    return QM_OK;
}

int32_t qmo_gate_up_swiglu_rows(const uint16_t* input, const uint16_t* gate_weight, const uint16_t* up_weight,
                                uint16_t* output, int32_t rows, int32_t hidden, int32_t intermediate,
                                int32_t n_threads) {
    if (!input || !gate_weight || !up_weight || !output) return QM_ERR_NULL;
    if (rows < 0 || hidden < 0 || intermediate < 0) return QM_ERR_ARGUMENT;
    for (int r = 0; r < rows; ++r) {
        const int32_t rc = qmo_gate_up_swiglu_m1(input + static_cast<int64_t>(r) * hidden, gate_weight, up_weight,
                                                 output + static_cast<int64_t>(r) * intermediate, hidden, intermediate,
                                                 n_threads);
        if (rc != QM_OK) return rc;
    }
    return QM_OK;
}

}  // extern "C"
