// Shared device helpers and launch parameter blocks for the gfx950 decoding-attention kernels.
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>
#include <stdint.h>

#include <type_traits>

namespace da {

constexpr int kWave = 64;          // CDNA4 wavefront width
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kNegBig = -1.0e30f;  // finite stand-in for -inf as the initial running maximum

struct f16_tag {};
struct bf16_tag {};

typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// Per-dtype element arithmetic on packed pairs held in a 32-bit register.
template <typename Tag>
struct Elem;

template <>
struct Elem<f16_tag> {
    // acc + a.lo*b.lo + a.hi*b.hi with fp32 accumulation (v_dot2_f32_f16)
    static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), acc, false);
    }
    static __device__ __forceinline__ float lo(uint32_t a) { return (float)__builtin_bit_cast(f16x2, a)[0]; }
    static __device__ __forceinline__ float hi(uint32_t a) { return (float)__builtin_bit_cast(f16x2, a)[1]; }
    // round-to-nearest-even, the reference's __float2half
    static __device__ __forceinline__ uint16_t from_f32(float f) {
        _Float16 h = (_Float16)f;
        return __builtin_bit_cast(uint16_t, h);
    }
    // two values rounded and packed (lo in bits 0 .. 15) by one instruction, v_cvt_pk_f16_f32
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        const f32x2 v = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
    }
    // (lo * s, hi * s) rounded and packed: the mixed-precision multiply-adds write the two halves of the result, one
    // instruction a value, each product rounded once
    static __device__ __forceinline__ uint32_t pack2_scaled(float lo, float hi, float s) {
        uint32_t r;
        asm("v_fma_mixlo_f16 %0, %1, %2, 0" : "=v"(r) : "v"(lo), "v"(s));
        asm("v_fma_mixhi_f16 %0, %1, %2, 0" : "+v"(r) : "v"(hi), "v"(s));
        return r;
    }
};

template <>
struct Elem<bf16_tag> {
    static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), acc,
                                               false);
    }
    static __device__ __forceinline__ float lo(uint32_t a) { return __uint_as_float(a << 16); }
    static __device__ __forceinline__ float hi(uint32_t a) { return __uint_as_float(a & 0xffff0000u); }
    // round-to-nearest-even, the reference's __float2bfloat16 (gfx950 converts in hardware, v_cvt_pk_bf16_f32; a NaN
    // stays a NaN)
    static __device__ __forceinline__ uint16_t from_f32(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }
    // two values rounded and packed (lo in bits 0 .. 15) by one instruction
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        const f32x2 v = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
    }
    // (lo * s, hi * s) rounded and packed
    static __device__ __forceinline__ uint32_t pack2_scaled(float lo, float hi, float s) { return pack2(lo * s, hi * s); }
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Maximum of a value with that of the lane 16 (32) positions away, lane ^ 16 (lane ^ 32), through the row and
// half-wave swap instructions: plain vector ALU work, no trip through the LDS crossbar as a shuffle makes.
__device__ __forceinline__ float max_xor16(float x) {
    const auto r = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(unsigned, x), __builtin_bit_cast(unsigned, x),
                                                    false, false);
    const unsigned r0 = r[0], r1 = r[1];  // (element copies first: a bit cast straight from r[1] reads r[0])
    return fmaxf(__builtin_bit_cast(float, r0), __builtin_bit_cast(float, r1));
}
__device__ __forceinline__ float max_xor32(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned, x), __builtin_bit_cast(unsigned, x),
                                                    false, false);
    const unsigned r0 = r[0], r1 = r[1];  // (element copies first: a bit cast straight from r[1] reads r[0])
    return fmaxf(__builtin_bit_cast(float, r0), __builtin_bit_cast(float, r1));
}

// A probability as the second matrix product will see it.  bf16 keeps 8 significant bits, so the rounded
// probabilities of a row no longer sum to the fp32 denominator; with the denominator summed from the rounded values
// the weights sum to one again, and the rounding errors enter as w (v - o) instead of w v -- what matters when few
// tokens carry the weight (steep ALiBi slopes, short sequences).  fp16's 11 bits are below the output rounding
// either way and are left alone.
template <typename Tag>
__device__ __forceinline__ float as_second_operand(float p) {
    if constexpr (std::is_same<Tag, bf16_tag>::value)
        return (float)(__bf16)p;
    else
        return p;
}

// 16 bytes of K or V from global memory, marked non-temporal: every K/V row is read once per call, and a plain
// streaming read of this GPU's HBM runs at 6.2-6.3 TB/s with ordinary loads and at 7.0-7.1 TB/s with this hint (the
// lines are not kept in the caches on their way through).
__device__ __forceinline__ uint4 stream_load16(const void* p) {
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}

// Formats of an 8-bit K/V cache (template argument KV8 of the kernels; 0 = 16-bit K/V).
constexpr int kKvFp8 = 1;   // OCP e4m3
constexpr int kKvInt8 = 2;  // two's-complement integers
// Four-bit integers (two's complement, -8 .. 7), two to a byte, element 2 i in the low half of byte i.  The kernels
// address such a cache as if it held one byte per element: the host hands them TWICE the buffer's address
// (SweepParams::k and ::v), all their row, head and lane arithmetic is the int8 arithmetic on those doubled addresses,
// and the load halves the address again (kv4_load8 / kv4_load16; every address the kernels form is even); the
// conversion to the compute type takes the nibbles straight to 16-bit values (int4x8_to_16).
constexpr int kKvInt4 = 3;
// Flag on top of a format (grouped kernel's template argument only): every (token, KV head) row carries its own
// (scale, zero) pair, element = scale * (integer - zero), instead of one factor per KV head (SweepParams::k_tok).
constexpr int kKvPerToken = 8;
// ... and on top of that: one pair per run of 64 elements of the row instead of one per row (head dims of 128 and 256:
// two and four pairs; SweepParams::k_tok then holds [rows, head_k, dim / 64, 2] floats).
constexpr int kKvGroup64 = 16;

// Eight FP8 (OCP e4m3) values -> eight 16-bit elements of the compute type.  Both conversions are exact (e4m3
// has 3 mantissa bits and |x| <= 448), so an FP8 K/V cache feeds the same arithmetic as a 16-bit one.
template <typename Tag>
__device__ __forceinline__ uint4 fp8x8_to_16(uint2 w) {
    uint4 r;
    if constexpr (std::is_same<Tag, f16_tag>::value) {
        r.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8((int)w.x, 1.0f, false));
        r.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8((int)w.x, 1.0f, true));
        r.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8((int)w.y, 1.0f, false));
        r.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8((int)w.y, 1.0f, true));
    } else {
        r.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)w.x, 1.0f, false));
        r.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)w.x, 1.0f, true));
        r.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)w.y, 1.0f, false));
        r.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)w.y, 1.0f, true));
    }
    return r;
}

// Four int8 values -> four 16-bit elements of the compute type, exactly (|x| <= 128 fits the 8 significant bits
// of bf16).  One conversion instruction per element: the sub-dword addressing of the vector ALU picks byte k of the
// word, sign-extends it, and (fp16) writes the result into one half of the destination register; bf16 goes through
// fp32, whose upper half is the bf16 value, and one byte permute packs a pair.
template <typename Tag>
__device__ __forceinline__ uint2 int8x4_to_16(uint32_t w) {
    uint2 r;
    if constexpr (std::is_same<Tag, f16_tag>::value) {
        asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_0" : "=v"(r.x) : "v"(w));
        asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_1" : "+v"(r.x) : "v"(w));
        asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_2" : "=v"(r.y) : "v"(w));
        asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_3" : "+v"(r.y) : "v"(w));
    } else {
        // (the compiler turns each cast into v_cvt_f32_i32 with a sign-extended byte operand)
        const float f0 = (float)(int8_t)(w), f1 = (float)(int8_t)(w >> 8);
        const float f2 = (float)(int8_t)(w >> 16), f3 = (float)(int8_t)(w >> 24);
        // v_perm_b32 picks result bytes from {first operand, second operand}: selector 0..3 = bytes of the second,
        // 4..7 = bytes of the first
        r.x = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, f1), __builtin_bit_cast(uint32_t, f0), 0x07060302u);
        r.y = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, f3), __builtin_bit_cast(uint32_t, f2), 0x07060302u);
    }
    return r;
}

// Factor by which int4x8_to_16 scales its values (the kernels divide it out of the per-head factors, exactly).
constexpr float kInt4Widening = 16.0f;
// Eight four-bit integers (one 32-bit word, element i in bits 4 i .. 4 i + 3, two's complement) -> eight 16-bit
// elements of the compute type holding SIXTEEN TIMES their values, in element order.  A nibble moved to the upper half
// of a byte whose lower half is zero is the signed byte 16 n, so two masks (and one shift) turn the word into the even
// elements' bytes and the odd elements' bytes, and from there on it is the int8 conversion: about 1.4 (fp16) and 1.9
// (bf16) vector instructions per element.  The factor 16 is a power of two: every product and sum downstream is the
// exact multiple, and dividing the per-head factors by it gives the int8 cache's results bit for bit.
template <typename Tag>
__device__ __forceinline__ uint4 int4x8_to_16(uint32_t w) {
    const uint32_t odd = w & 0xF0F0F0F0u;          // byte j: 16 x element 2 j + 1
    const uint32_t even = (w << 4) & 0xF0F0F0F0u;  // byte j: 16 x element 2 j
    uint4 r;
    if constexpr (std::is_same<Tag, f16_tag>::value) {
#define DA_CVT_PAIR(dst, B)                                                                                               \
    asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_" #B : "=v"(dst) : "v"(even)); \
    asm("v_cvt_f16_i16_sdwa %0, sext(%1) dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_" #B : "+v"(dst) : "v"(odd));
        DA_CVT_PAIR(r.x, 0)
        DA_CVT_PAIR(r.y, 1)
        DA_CVT_PAIR(r.z, 2)
        DA_CVT_PAIR(r.w, 3)
#undef DA_CVT_PAIR
    } else {
        auto pair = [&](int sh) {
            const float lo = (float)(int8_t)(even >> sh), hi = (float)(int8_t)(odd >> sh);
            return __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, hi), __builtin_bit_cast(uint32_t, lo), 0x07060302u);
        };
        r.x = pair(0);
        r.y = pair(8);
        r.z = pair(16);
        r.w = pair(24);
    }
    return r;
}
// The matrix kernel's conversion of the same word: eight 16-bit elements holding kInt4Bias + n, in the order
// kInt4Order (slot s holds element kInt4Order[s]: the low halves of the four result words are nibbles 0 .. 3, the
// high halves nibbles 4 .. 7).  With the top bit of every nibble flipped, n + 8 = 0 .. 15 placed in the four leading
// mantissa bits of 16.0 is the number 16 + (n + 8) exactly, in fp16 and in bf16: one XOR per word, then a shift and an
// AND-OR (one instruction) per pair, 1.1 vector instructions per element.  The kernel takes the bias back out of its sums (q . (24 + n)
// = q . n + 24 sum(q); sum_t p (24 + n) = sum_t p n + 24 sum_t p) and undoes the order where it matters.
constexpr float kInt4Bias = 24.0f;
template <typename Tag>
__device__ __forceinline__ uint32_t int4_biased_one() {
    uint32_t one = std::is_same<Tag, f16_tag>::value ? 0x4C004C00u : 0x41804180u;  // 16.0 in both halves
    asm("" : "+v"(one));  // (kept in a vector register: see int4x8_biased)
    return one;
}
template <typename Tag>
__device__ __forceinline__ uint4 int4x8_biased(uint32_t w, uint32_t one) {
    constexpr bool kHalf = std::is_same<Tag, f16_tag>::value;
    // the four leading mantissa bits of both halves, and 16.0 in both halves (fp16 0x4C00: bits 6 .. 9; bf16 0x4180:
    // bits 3 .. 6)
    constexpr uint32_t kMask = kHalf ? 0x03C003C0u : 0x00780078u;
    constexpr int kAt = kHalf ? 6 : 3;  // where nibble 0 has to go
    const uint32_t x = w ^ 0x88888888u;
    // (shifted & mask) | 16.0 as one instruction: the mask travels in a scalar register and 16.0 (`one`, from
    // int4_biased_one, once per kernel) in a vector register: the instruction's encoding takes no literal constants,
    // and one scalar operand at most
    auto place = [&](uint32_t shifted) {
        uint32_t r;
        asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(shifted), "s"(kMask), "v"(one));
        return r;
    };
    uint4 r;
    r.x = place(x << kAt);
    r.y = place(kAt >= 4 ? x << (kAt - 4) : x >> (4 - kAt));
    r.z = place(x >> (8 - kAt));
    r.w = place(x >> (12 - kAt));
    return r;
}

// Sixteen (eight) elements of an int4 cache at the doubled address `vptr` (see kKvInt4): the packed words, each in
// the slot where the 8-bit formats keep the eight bytes of the same elements (the other word of the pair is unused).
// The halved address is cast to the global address space by hand: an address that went through integer arithmetic
// is a generic one to the compiler, and a generic (flat) load counts against the LDS counter as well, so that every
// wait for an LDS read would also wait for the K/V loads in flight.
__device__ __forceinline__ uint4 kv4_load16(const void* vptr) {
    typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
    typedef const u32x2 __attribute__((address_space(1))) * global_u32x2_ptr;
    const u32x2 w = *(global_u32x2_ptr)(reinterpret_cast<uintptr_t>(vptr) >> 1);
    return make_uint4(w.x, 0u, w.y, 0u);
}
__device__ __forceinline__ uint2 kv4_load8(const void* vptr) {
    typedef const uint32_t __attribute__((address_space(1))) * global_u32_ptr;
    return make_uint2(*(global_u32_ptr)(reinterpret_cast<uintptr_t>(vptr) >> 1), 0u);
}

// Eight elements of an 8-bit K/V cache of format FMT -> eight 16-bit elements of the compute type (an int4 cache's
// eight elements are the nibbles of w.x, and come out scaled by kInt4Widening).
template <typename Tag, int FMT>
__device__ __forceinline__ uint4 kv8x8_to_16(uint2 w) {
    static_assert(FMT == kKvFp8 || FMT == kKvInt8 || FMT == kKvInt4, "8-bit K/V format");
    if constexpr (FMT == kKvFp8) {
        return fp8x8_to_16<Tag>(w);
    } else if constexpr (FMT == kKvInt4) {
        return int4x8_to_16<Tag>(w.x);
    } else {
        const uint2 a = int8x4_to_16<Tag>(w.x), b = int8x4_to_16<Tag>(w.y);
        return make_uint4(a.x, a.y, b.x, b.y);
    }
}
// What the conversion multiplied the elements by, inverted (divided out of the per-head factors).
template <int FMT>
__device__ __forceinline__ float kv_widening_inverse() {
    return FMT == kKvInt4 ? 1.0f / kInt4Widening : 1.0f;
}

// f(integral_constant<int, B>), ..., f(integral_constant<int, E-1>): a loop whose index is a constant
// expression in the body (needed for instruction offset fields and wait counts in inline assembly).
template <int B, int E, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        static_for<B + 1, E>(f);
    }
}

// Butterfly sum over groups of G adjacent lanes (G a power of two <= 16) with DPP lane
// permutes; every lane of the group ends with the group's total.
template <int G>
__device__ __forceinline__ float group_sum(float x) {
    if constexpr (G >= 2) {  // quad_perm [1,0,3,2]
        x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0xB1, 0xF, 0xF, true));
    }
    if constexpr (G >= 4) {  // quad_perm [2,3,0,1]
        x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x4E, 0xF, 0xF, true));
    }
    if constexpr (G >= 8) {  // row_half_mirror: quads are uniform by now, so i -> 7-i swaps the two quads
        x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x141, 0xF, 0xF, true));
    }
    if constexpr (G >= 16) {  // row_mirror: halves are uniform, i -> 15-i swaps them
        x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x140, 0xF, 0xF, true));
    }
    return x;
}

// Argument block of the sweep kernels (passed by value).
struct SweepParams {
    const void* q;            // [batch, head_q, dim]
    const void* k;            // [total_k, head_k, dim]
    const void* v;            // [total_k, head_k, dim_v], or k when V is the leading columns of K
    void* o;                  // [batch, head_q, dim_v]
    const int32_t* cu_seq_k;  // [batch + 1]
    float* ws_o;              // [batch, head_q, nsplit, dim_v] un-normalised partial outputs
    float* ws_ml;             // [batch, head_q, nsplit, 2] running maximum (log2 units) and denominator
    const float* slopes;      // [head_q] ALiBi slopes or null for the closed form
    int64_t k_row;            // elements between consecutive tokens of K
    int64_t v_row;            // same for V
    int v_head;               // elements between KV heads of V
    int head_q, head_k, ratio;
    int groups;               // work-groups per KV head (ceil(ratio / heads per work-group))
    int nsplit, chunk;        // sequence splits and tokens per split
    int nat_partials;         // latent kernels: split partials as normalised 16-bit block records (nat_block below)
    float scale_log2;         // softmax scale * log2(e)
    int is_alibi;
    // Paged K/V (block_table != null): k and v are page pools [pages, page_size, head_k, dim(_v)], token j of
    // sequence b is row j % page_size of page block_table[b, j / page_size]; cu_seq_k is null and seq_lens
    // gives the lengths.  page_size is a power of two.
    const int32_t* block_table;  // [batch, max_blocks]
    const int32_t* seq_lens;     // [batch]
    int page_shift, max_blocks;
    int64_t k_page, v_page;      // elements between consecutive pages of K and of V
    // De-quantisation factors of an FP8 K/V cache, one per KV head (null = 1): K = k_scale[hk] * fp8 value.
    // The kernels fold k_scale into the softmax scale and v_scale into the final normalisation.
    const float* k_scale;
    const float* v_scale;
    // Per-token asymmetric quantisation (grouped kernel, int4): (scale, zero) float pairs per (token, KV head), laid
    // out like the rows they belong to ([total_k, head_k, 2], or [pages, page_size, head_k, 2] dense);
    // K[t, hk, c] = k_tok[t, hk].scale * (integer - k_tok[t, hk].zero), V likewise.  Null: per-head factors above.
    const float* k_tok;
    const float* v_tok;
    // Balanced form of the grouped-head kernel's grid (flat_wgs == 0: off).  The sequences lie end to end on one line
    // measured in units of flat_unit tokens (1 for packed K/V, where the line is cu_seq_k itself; 32 for paged K/V,
    // where every sequence is rounded up to whole units so that shares start on tile boundaries); flat_cu[b] is the
    // position of sequence b on the line ([batch + 1] entries).  Each of flat_wgs work-groups takes an equal share of
    // the line, flat_share() units, which the kernels derive from the line's length flat_cu[batch] themselves: the
    // host never needs the token count.
    int flat_wgs;
    int flat_step, flat_min;  // a share is a multiple of flat_step units and at least flat_min
    int flat_unit;
    const int32_t* flat_cu;
    int batch;
};

__device__ __forceinline__ float head_scale(const float* scales, int hk) { return scales ? scales[hk] : 1.0f; }

struct ReduceParams {
    void* o;
    const int32_t* cu_seq_k;
    const int32_t* seq_lens;  // lengths when cu_seq_k is null (paged K/V)
    const float* ws_o;
    const float* ws_ml;
    int head_q, dim_v, nsplit, chunk;
    // balanced form of the sweep's grid (flat_wgs > 0): work-groups along the line, share granularity and minimum, the
    // sequences' positions on the line (see SweepParams)
    int flat_wgs, flat_step, flat_min;
    const int32_t* flat_cu;
    int batch;
    // the workspace is small (cache-resident): request the first partials before the sequence's length is known
    int early;
    // the partial outputs are normalised (divided by their denominators) and stored as 16-bit values of the output
    // type from the start of ws_o, in the order the matrix instruction leaves them in registers and with their
    // (m, l) pairs beside them (nat_block below; ws_ml is not used), instead of un-normalised fp32 by rows (the
    // pipelined latent kernel: its partials, 128 heads x 512 columns per split, are most of the traffic that
    // splitting adds)
    int half_partials;
    int ratio, groups, nat_blocks;  // (half_partials) query heads per KV head, work-groups per KV head, nat_blocks()
    int nat_waves;                  // (half_partials) waves, i.e. blocks of 32 heads, per work-group of the sweep
};

// Normalised 16-bit partials of the latent kernels (dim_v = 512).  A wave of those kernels owns 32 query heads (a
// block; block id = (KV head * groups + group) * waves per work-group + wave, rows past the group's last head are
// dead), and after the last matrix step lane (n, half) holds, for each 32-column tile c = 0 .. 15 and r4 = 0 .. 3, the
// four columns 32 c + 8 r4 + 4 half .. + 3 of head n.  The wave stores them as they lie, 16 bytes a lane (the pieces
// r4 = 2 rp and 2 rp + 1 together): one split's partial of one block is a record of 32 runs of 1 KiB, run 2 c + rp
// holding lane after lane, followed by the 32 rows' (running maximum, denominator) pairs, so that everything the
// merge reads of 32 rows and one split lies together and both sides move 16 bytes a lane.  In 8-byte units:
constexpr int kNatBlockUnits = 64 * 64 + 32;  // a block record: 32 KiB of partial outputs + 32 float2
__host__ __device__ inline int nat_blocks(int head_k, int groups, int waves) { return head_k * groups * waves; }
// start of the record of block blk, split s of sequence b
__device__ __forceinline__ size_t nat_block(size_t b, int nsplit, int s, int nblk, int blk) {
    return ((b * nsplit + s) * nblk + blk) * (size_t)kNatBlockUnits;
}
// columns 4 c4 .. 4 c4 + 3 of row n, relative to the record's start: column bits 5.. = c, 4 = rp, 3 = which half of
// the lane's 16 bytes, 2 = half-wave
__device__ __forceinline__ int nat_piece(int c4, int n) {
    return ((c4 >> 2) * 64 + (c4 & 1) * 32 + n) * 2 + ((c4 >> 1) & 1);
}
// (m, l) of row n, relative to the record's start
__device__ __forceinline__ int nat_ml(int n) { return 64 * 64 + n; }
// bytes of one sequence split's records
__host__ __device__ inline size_t nat_split_bytes(int nblk) { return (size_t)nblk * kNatBlockUnits * 8; }

// Balanced grid: units per work-group for a line of `total` units cut into `wgs` shares.
__host__ __device__ inline int flat_share(long long total, int wgs, int step, int mn) {
    long long t = (total + wgs - 1) / wgs;
    t = (t + step - 1) / step * step;
    const long long floor_t = mn > step ? mn : step;
    return (int)(t > floor_t ? t : floor_t);
}
// Partial slot of (sequence b, share i): consecutive sequences may meet in one share, so the slots of a batch are
// numbered share + sequence -- strictly increasing along the line, below wgs + batch -- which needs no knowledge of the
// share length when the workspace is sized.
__host__ __device__ inline size_t flat_slots(int wgs, size_t batch) { return (size_t)wgs + batch; }

// First token (row of the packed K/V buffers) and length of sequence b; paged sequences start at row 0 of their
// own pages.
__device__ __forceinline__ void seq_range(const SweepParams& p, int b, int& start, int& len) {
    if (p.block_table) {
        start = 0;
        len = p.seq_lens[b];
    } else {
        start = p.cu_seq_k[b];
        len = p.cu_seq_k[b + 1] - start;
    }
}

// Element offsets (head 0, column 0) of token j of sequence b in the K and V buffers.  The lookup comes in two
// steps so that a kernel can fetch the page id early and do the arithmetic when it needs the address.
struct RowRef {
    int64_t k, v;
};
__device__ __forceinline__ int page_of(const SweepParams& p, int b, int j) {
    if (p.block_table == nullptr) return 0;
    // The table is read through the constant address space: nothing writes it while the kernel runs, and that
    // lets a wave-uniform lookup become a scalar load even after assembly statements that clobber memory.
    typedef const int32_t __attribute__((address_space(4))) * const_i32;
    const const_i32 table = (const_i32)(uintptr_t)p.block_table;
    return table[(int64_t)b * p.max_blocks + (j >> p.page_shift)];
}
__device__ __forceinline__ RowRef row_in_page(const SweepParams& p, int start, int j, int page) {
    if (p.block_table == nullptr) return {(int64_t)(start + j) * p.k_row, (int64_t)(start + j) * p.v_row};
    const int r = j & ((1 << p.page_shift) - 1);
    return {(int64_t)page * p.k_page + (int64_t)r * p.k_row, (int64_t)page * p.v_page + (int64_t)r * p.v_row};
}
__device__ __forceinline__ RowRef row_ref(const SweepParams& p, int b, int start, int j) {
    return row_in_page(p, start, j, page_of(p, b, j));
}

// An empty sequence still owns output rows: when the sequence is not split, its work-group stores zeros for
// its heads (n_ranges runs of nheads consecutive heads, range_stride apart); otherwise the merge kernel does.
template <int DV>
__device__ __forceinline__ void zero_rows(const SweepParams& p, int b, int h_first, int nheads, int n_ranges,
                                          int range_stride) {
    uint16_t* const o16 = reinterpret_cast<uint16_t*>(p.o);
    for (int it = threadIdx.x; it < n_ranges * nheads * DV; it += blockDim.x) {
        const int col = it % DV;
        const int hh = (it / DV) % nheads;
        const int rg = it / (DV * nheads);
        o16[((size_t)b * p.head_q + h_first + rg * range_stride + hh) * DV + col] = 0;
    }
}

__device__ __forceinline__ float alibi_slope_log2(const float* slopes, int h, int head_q) {
    // closed form 2^(-8(h+1)/head_q); a slope array overrides it
    float s = slopes ? slopes[h] : fast_exp2(-8.0f * (float)(h + 1) / (float)head_q);
    return s * kLog2e;
}

// Raise a kernel's dynamic LDS limit once per device (the attribute belongs to the function on the current
// device, and one process may drive several).  `done` is the caller's per-kernel bit mask of devices served.
inline hipError_t ensure_lds_limit(const void* kernel, size_t lds_bytes, std::atomic<uint64_t>& done) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const uint64_t bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);  // (a failure is retried by the next call)
    return e;
}

}  // namespace da
