// qm_device.h — device-side helpers shared by the gfx950 kernels (wave64 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/qm_attn.h"

namespace qm {

constexpr int kDim = 128;         // head dimension of every supported model family
constexpr int kTile = 16;         // tokens per K/V tile = tokens per native page
constexpr float kLog2e = 1.4426950408889634f;

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

// bf16 <-> f32 exactly as the reference does it (R17:15024-15056): widening is a shift,
// narrowing is round-to-nearest-even on the bit pattern with NaNs quieted.
__device__ __forceinline__ float bf2f(uint16_t v) {
    return __uint_as_float(static_cast<uint32_t>(v) << 16);
}

__device__ __forceinline__ uint16_t f2bf(float value) {
    // v_cvt_pk_bf16_f32 gives, for every one of the 2^32 fp32 bit patterns, the bits of the reference's integer
    // sequence (add 0x7fff + the lowest kept bit, shift; a NaN quieted with its payload kept): compared exhaustively
    // on the device.  One instruction instead of six and a branch.
    uint32_t packed;
    asm("v_cvt_pk_bf16_f32 %0, %1, %1" : "=v"(packed) : "v"(value));
    return static_cast<uint16_t>(packed);
}

// Round an fp32 value to the nearest bf16 and widen it again (hardware RNE convert).
__device__ __forceinline__ float round_bf16(float x) {
    return static_cast<float>(static_cast<__bf16>(x));
}

// One rounding with one v_cvt_pk_bf16_f32 and nothing to take apart: (0, x) converts to bf16(x) in the
// upper half of the register over zeros, which is the rounded value as fp32.
__device__ __forceinline__ float round_bf16_single(float x) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t in = {0.0f, x};
    return __uint_as_float(__builtin_bit_cast(uint32_t, __builtin_convertvector(in, bf16x2_t)));
}

// Two roundings with one v_cvt_pk_bf16_f32.
__device__ __forceinline__ void round_bf16_pair(float a, float b, float& ra, float& rb) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t in = {a, b};
    const bf16x2_t packed = __builtin_convertvector(in, bf16x2_t);
    const uint32_t bits = __builtin_bit_cast(uint32_t, packed);
    ra = __uint_as_float(bits << 16);
    rb = __uint_as_float(bits & 0xffff0000U);
}

// (a, b) -> packed bf16 pair, a in the low half (one v_cvt_pk_bf16_f32, round to nearest even).
__device__ __forceinline__ uint32_t pack_bf16_pair(float a, float b) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t in = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(in, bf16x2_t));
}

__device__ __forceinline__ float lo_bf16(uint32_t packed) { return __uint_as_float(packed << 16); }
__device__ __forceinline__ float hi_bf16(uint32_t packed) { return __uint_as_float(packed & 0xffff0000U); }

// acc + a.x*b.x + a.y*b.y on packed bf16 pairs (v_dot2c_f32_bf16).
__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a),
                                           __builtin_bit_cast(bf16x2_t, b), acc, false);
}

// A kernel's arguments are scalar loads of the launch's argument block, and the compiler requests each where it is
// first used: a block then waits for memory once per group of arguments, one round trip after the other, before it
// can ask for its first operand (1 300 cycles each on this chip for lines that no wave has read yet).  Called first
// thing in a kernel with its by-value arguments, this asks for one word of every 32 bytes of all of them at once and
// waits once; what the kernel reads later comes from the scalar cache.
template <class T>
__device__ __forceinline__ uint32_t argument_words(const T& argument) {
    static_assert(sizeof(T) % 4 == 0, "whole 32-bit words");
    struct Words { uint32_t w[sizeof(T) / 4]; };
    const Words words = __builtin_bit_cast(Words, argument);
    uint32_t all = words.w[sizeof(T) / 4 - 1];
#pragma unroll
    for (size_t i = 0; i < sizeof(T) / 4; i += 8) all ^= words.w[i];
    return all;
}
template <class... T>
__device__ __forceinline__ void request_arguments(const T&... arguments) {
    const uint32_t all = (argument_words(arguments) ^ ...);
    asm volatile("" :: "s"(all));
}

// 2^x with the bare v_exp_f32 instruction (inputs here are <= 0 or -inf).
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// DPP row rotate: lane i of each 16-lane row reads lane (i - n) mod 16 of its row.
template <int N>
__device__ __forceinline__ float row_ror(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x120 + N, 0xf, 0xf, false));
}

// Sum over the 16 lanes of a DPP row; every lane of the row receives the total.
__device__ __forceinline__ float row16_allreduce_sum(float v) {
    v += row_ror<8>(v);
    v += row_ror<4>(v);
    v += row_ror<2>(v);
    v += row_ror<1>(v);
    return v;
}

// Logical-token -> page mapping precomputed on the host (a shift when page_size is a power
// of two, page 0 when the sequence has a single page).
struct PageMap {
    int page_size;
    int shift;      // log2(page_size) or -1
    int max_pages;
};

__host__ __device__ inline PageMap make_page_map(int page_size, int max_pages) {
    PageMap m;
    m.page_size = page_size;
    m.max_pages = max_pages;
    m.shift = -1;
    for (int s = 0; s < 31; ++s) {
        if ((1 << s) == page_size) m.shift = s;
    }
    return m;
}

__device__ __forceinline__ int page_of(const PageMap& pm, int token) {
    if (pm.shift >= 0) return token >> pm.shift;
    if (pm.max_pages == 1) return token < pm.page_size ? 0 : 1;
    return token / pm.page_size;
}

// Element offset of token `first_token` of kv head `head` (the addressing rule documented at
// qm_kv_cache), or -1 with a status bit if the page is out of range.
__device__ __forceinline__ int64_t tile_offset(const qm_kv_cache& c, const PageMap& pm,
                                               const int32_t* page_table, int first_token,
                                               int head, uint32_t* status) {
    const int page = page_of(pm, first_token);
    if (page >= pm.max_pages) {
        if (status) atomicOr(status, QM_STATUS_BAD_POSITION);
        return -1;
    }
    const int phys = page_table ? page_table[page] : page;
    if (phys < 0 || phys >= c.n_pages) {
        if (status) atomicOr(status, QM_STATUS_BAD_PAGE);
        return -1;
    }
    return static_cast<int64_t>(phys) * c.stride_page + static_cast<int64_t>(head) * c.stride_head
         + static_cast<int64_t>(first_token - page * pm.page_size) * kDim;
}

// The reference's wave reduction, value += shfl_down(value, offset, 32) for offset 16, 8, 4, 2, 1 (R17:9359-9364,
// 15059-15075), for the lane whose result is used: lane 0 of each 32-lane half of the wave ends with the sum that
// loop leaves there, formed by the same additions in the same order (other lanes end with something else).
// No LDS traffic: the exchange between the two 16-lane rows is v_permlane16_swap, the rest are DPP row shifts,
// whose lanes beyond the row read zero.
__device__ __forceinline__ float half_wave_tree_sum(float v) {
    const auto rows = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(rows[0]) + __uint_as_float(rows[1]);      // every lane: its own value + that of lane ^ 16
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x108, 0xf, 0xf, true));   // row_shl:8
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x104, 0xf, 0xf, true));   // row_shl:4
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x102, 0xf, 0xf, true));   // row_shl:2
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x101, 0xf, 0xf, true));   // row_shl:1
    return v;
}

// block_reduce_sum / talker_block_sum of the reference (R17:8233-8274, 15102-15148) for a block of 256
// threads: eight 32-lane shfl_down trees, then one tree over the eight results.  sh_waves: 8 floats,
// sh_total: 1 float of LDS; the total is valid in every thread.
__device__ __forceinline__ float block_sum_256_like_reference(float value, float* sh_waves, float* sh_total) {
    const int tid = threadIdx.x;
    value = half_wave_tree_sum(value);
    if ((tid & 31) == 0) sh_waves[tid >> 5] = value;
    __syncthreads();
    if (tid < 32) {
        float v = tid < 8 ? sh_waves[tid] : 0.0f;
        v = half_wave_tree_sum(v);
        if (tid == 0) *sh_total = v;
    }
    __syncthreads();
    return *sh_total;
}

}  // namespace qm
