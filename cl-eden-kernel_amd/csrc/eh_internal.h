// Internal declarations shared by the translation units of libedenhip.so.
// gfx950 (MI355X) only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "eden_hip.h"

namespace eh {

// ---------------------------------------------------------------- errors
void set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
int hip_fail(hipError_t e, const char *what);  // records the text, returns EH_DEVICE_FAILURE

#define EH_HIP(call)                                          \
    do {                                                      \
        hipError_t eh_e_ = (call);                            \
        if (eh_e_ != hipSuccess) return ::eh::hip_fail(eh_e_, #call); \
    } while (0)

#define EH_REQUIRE(cond, ...)               \
    do {                                    \
        if (!(cond)) {                      \
            ::eh::set_error(__VA_ARGS__);   \
            return EH_INVALID_PARAMS;       \
        }                                   \
    } while (0)

// ---------------------------------------------------------------- requant
// Integer requantization as the reference's generic kernels do it
// (gpu/common/CLKernels.hpp:120-170): saturating rounding doubling high mul,
// rounding divide by a power of two, output zero point, activation clamp.
struct RequantDev {
    int32_t multiplier;
    int32_t left_shift;
    int32_t right_shift;
    int32_t mask;  // (1 << right_shift) - 1
    int32_t half;  // mask >> 1
    int32_t zp_out;
    int32_t act_min;
    int32_t act_max;
    // single-shift form (see requant_u8_fast); valid when `fast` is set (2: the sign test may be skipped too)
    int32_t fast;
    int32_t fast_shift;        // right_shift - 1
    uint32_t pos_lo, pos_hi;   // 64-bit rounding term for accumulators >= 0
    uint32_t neg_lo, neg_hi;   // the same for accumulators < 0
    int32_t lo_scaled, hi_scaled;  // the clamp of the single-shift form applied before its shift (see requant4_fast)
    // per-output-channel quantization (int8 weights with one scale per channel): device arrays indexed by the
    // problem's own channel number, or null; when set they replace multiplier and shift above
    const int32_t *pc_multiplier;
    const int32_t *pc_shift;
};

__host__ __device__ __forceinline__ int32_t requant_core(int32_t acc, const RequantDev &r) {
    // x * (1 << ls) wraps like the int32 multiply of the reference kernels
    const int32_t x = (int32_t)((uint32_t)acc << r.left_shift);
    // (ab + nudge) / 2^31 with nudge = ab >= 0 ? 2^30 : 1 - 2^30 and C truncation
    // is floor((ab + 2^30) / 2^31) for every ab; the multiplier is never
    // INT32_MIN (the host rejects negative multipliers), so no saturation case.
    const int64_t ab = (int64_t)x * (int64_t)r.multiplier + (1ll << 30);
    const int32_t v = (int32_t)(ab >> 31);
    // rounding divide by 2^rs: remainder > (mask >> 1) + (v < 0)
    const int32_t rem = v & r.mask;
    const int32_t thr = r.half - (v >> 31);
    return (v >> r.right_shift) + (rem > thr ? 1 : 0);
}

__host__ __device__ __forceinline__ uint32_t requant_u8(int32_t acc, const RequantDev &r) {
    int32_t v = requant_core(acc, r) + r.zp_out;
    v = v < r.act_min ? r.act_min : v;
    v = v > r.act_max ? r.act_max : v;
    return (uint32_t)v;
}

// One multiplier and shift per output channel (conv_per_channel_quantized,
// gpu/operators/cl_kernels/ConvolutionKernels.cpp:1317-1375): the two-step order with the
// channel's own parameters; shift > 0 is a left shift of the accumulator, as above.
__host__ __device__ __forceinline__ uint32_t requant_u8_channel(int32_t acc, int32_t multiplier, int32_t shift, const RequantDev &r) {
    const int32_t ls = shift > 0 ? shift : 0, rs = shift > 0 ? 0 : -shift;
    const int32_t x = (int32_t)((uint32_t)acc << ls);
    const int64_t ab = (int64_t)x * (int64_t)multiplier + (1ll << 30);
    int32_t v = (int32_t)(ab >> 31);
    const int32_t mask = (int32_t)((1u << rs) - 1u);
    const int32_t rem = v & mask;
    const int32_t thr = (mask >> 1) - (v >> 31);
    v = (v >> rs) + (rem > thr ? 1 : 0) + r.zp_out;
    v = v < r.act_min ? r.act_min : v;
    v = v > r.act_max ? r.act_max : v;
    return (uint32_t)v;
}

// The same function in one multiply-add and one shift, for left_shift == 0 and
// 1 <= right_shift <= 21.  With v = floor((xM + 2^30) / 2^31), h = 2^(rs-1) and
// s = -(v < 0), the rounding divide is floor((v + h + s) / 2^rs), and since h + s
// is an integer the two floors merge:
//     result + zp = floor((xM + 2^30 + (h + s + zp * 2^rs) * 2^31) / 2^(31 + rs)).
// s may be taken from the sign of x: where x < 0 but v = 0 (-2^30 <= xM < 0) the
// numerator stays inside [0, 2^(30 + rs)), so the result is 0 either way.  The
// quotient by 2^(31 + rs) with rs >= 1 only needs the high word of the sum.
__host__ __device__ __forceinline__ uint32_t requant_u8_fast(int32_t x, const RequantDev &r) {
    const bool neg = x < 0;
    const uint64_t term = ((uint64_t)(neg ? r.neg_hi : r.pos_hi) << 32) | (neg ? r.neg_lo : r.pos_lo);
    const int64_t t = (int64_t)x * (int64_t)r.multiplier + (int64_t)term;
    int32_t v = (int32_t)(t >> 32) >> r.fast_shift;
    v = v < r.act_min ? r.act_min : v;
    v = v > r.act_max ? r.act_max : v;
    return (uint32_t)v;
}

// Where the clamp floor is not below the output zero point (a fused ReLU-type activation),
// every negative accumulator ends on the floor whichever way its tie is broken (the quotient
// with the non-negative rounding term is still <= 0), so the sign test can go.
__host__ __device__ __forceinline__ uint32_t requant_u8_fast_relu(int32_t x, const RequantDev &r) {
    const int64_t term = (int64_t)(((uint64_t)r.pos_hi << 32) | r.pos_lo);
    const int64_t t = (int64_t)x * (int64_t)r.multiplier + term;
    int32_t v = (int32_t)(t >> 32) >> r.fast_shift;
#if defined(__HIP_DEVICE_COMPILE__)
    // act_min <= act_max always holds, so the clamp is a median of three (one instruction; the
    // compiler cannot assume the ordering and would emit max + min)
    int32_t o;
    asm("v_med3_i32 %0, %1, %2, %3" : "=v"(o) : "v"(v), "s"(r.act_min), "v"(r.act_max));
    return (uint32_t)o;
#else
    v = v < r.act_min ? r.act_min : v;
    v = v > r.act_max ? r.act_max : v;
    return (uint32_t)v;
#endif
}

// Four outputs of the single-shift form, packed into one word, lowest byte first, in three instructions each (MODE 2)
// or six (MODE 1).  `extra` is an addend that all four accumulators still lack (a pixel's row-sum term): it goes into
// the 64-bit rounding term as extra * M, once for every call that shares it, instead of into each accumulator, and the
// sign test of MODE 1 compares against -extra.  The clamp comes before the shift, on bounds scaled by 2^fs: floor is
// monotone, so clamp(h >> fs, a, b) == clamp(h, a << fs, (b << fs) | (2^fs - 1)) >> fs.  What is left to shift is
// non-negative and ends in 0 .. 255, so the shift writes its byte of the packed word directly (an SDWA destination
// select that keeps the other bytes).  Needs 0 <= act_min <= act_max <= 255, which the operators' entry points check.
template <int MODE>
__host__ __device__ __forceinline__ uint32_t requant4_fast(int32_t x0, int32_t x1, int32_t x2, int32_t x3, int32_t extra, const RequantDev &r) {
    static_assert(MODE == 1 || MODE == 2, "single-shift forms only");
    const int64_t pos = (int64_t)(((uint64_t)r.pos_hi << 32) | r.pos_lo) + (int64_t)extra * (int64_t)r.multiplier;
    const int64_t neg = pos - (1ll << 31);
    const int32_t zero = -extra;  // (extra is a sum of at most a few thousand byte products: no overflow)
    auto high = [&](int32_t x) {
        const int64_t term = (MODE == 1 && x < zero) ? neg : pos;
        const int32_t h = (int32_t)(((int64_t)x * (int64_t)r.multiplier + term) >> 32);
#if defined(__HIP_DEVICE_COMPILE__)
        int32_t o;
        asm("v_med3_i32 %0, %1, %2, %3" : "=v"(o) : "v"(h), "s"(r.lo_scaled), "v"(r.hi_scaled));
        return o;
#else
        return h < r.lo_scaled ? r.lo_scaled : h > r.hi_scaled ? r.hi_scaled : h;
#endif
    };
    const int32_t h0 = high(x0), h1 = high(x1), h2 = high(x2), h3 = high(x3);
#if defined(__HIP_DEVICE_COMPILE__)
    uint32_t w;
    asm("v_lshrrev_b32_sdwa %0, %1, %2 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:DWORD" : "=v"(w) : "v"(r.fast_shift), "v"(h0));
    asm("v_lshrrev_b32_sdwa %0, %1, %2 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(w) : "v"(r.fast_shift), "v"(h1));
    asm("v_lshrrev_b32_sdwa %0, %1, %2 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(w) : "v"(r.fast_shift), "v"(h2));
    asm("v_lshrrev_b32_sdwa %0, %1, %2 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(w) : "v"(r.fast_shift), "v"(h3));
    return w;
#else
    const int fs = r.fast_shift;
    return (uint32_t)(h0 >> fs) | ((uint32_t)(h1 >> fs) << 8) | ((uint32_t)(h2 >> fs) << 16) | ((uint32_t)(h3 >> fs) << 24);
#endif
}

// The single-shift form with a channel's own multiplier and shift (-20 <= shift <= -1; the host sets `fast` on a
// per-channel problem only when every channel is in that range).  The rounding term 2^30 + (1 + 2 zp) 2^(30 + rs)
// depends on the channel alone, so a thread that keeps its channels across many outputs computes it once.
// MODE 2 skips the sign test as requant_u8_fast_relu does.
template <int MODE>
__host__ __device__ __forceinline__ uint32_t requant_u8_channel_fast(int32_t x, int32_t multiplier, int32_t shift, const RequantDev &r) {
    const int32_t rs = -shift;
    const int64_t pos = (1ll << 30) + (int64_t)(1 + 2 * r.zp_out) * (1ll << (30 + rs));
    const int64_t term = (MODE != 2 && x < 0) ? pos - (1ll << 31) : pos;
    const int64_t t = (int64_t)x * (int64_t)multiplier + term;
    int32_t v = (int32_t)(t >> 32) >> (rs - 1);
    v = v < r.act_min ? r.act_min : v;
    v = v > r.act_max ? r.act_max : v;
    return (uint32_t)v;
}

// The same with the channel's terms from a table: `fs` = rs - 1 and `pos_hi` = (1 + 2 zp) 2^(rs - 2), the high word
// of the rounding term, whose low word is 2^30 for every rs >= 2.  For a negative accumulator the term is 2^31
// less: the low word gains bit 31 and the high word lends one.
template <int MODE>
__host__ __device__ __forceinline__ uint32_t requant_u8_channel_table(int32_t x, int32_t multiplier, int32_t fs, int32_t pos_hi,
                                                                      const RequantDev &r) {
    uint32_t lo = 0x40000000u;
    int32_t hi = pos_hi;
    if (MODE != 2) {
        lo |= (uint32_t)x & 0x80000000u;
        hi += x >> 31;
    }
    const int64_t t = (int64_t)x * (int64_t)multiplier + (int64_t)(((uint64_t)(uint32_t)hi << 32) | lo);
    int32_t v = (int32_t)(t >> 32) >> fs;
    v = v < r.act_min ? r.act_min : v;
    v = v > r.act_max ? r.act_max : v;
    return (uint32_t)v;
}

// high word of the table form's rounding term for a right shift rs >= 2
__host__ __device__ __forceinline__ int32_t channel_table_pos_hi(int32_t zp_out, int32_t rs) {
    return (int32_t)((uint32_t)(1 + 2 * zp_out) << (rs - 2));
}

// whether the single-shift form covers a channel's pair
inline bool channel_pair_is_fast(int32_t multiplier, int32_t shift, int32_t max_shift = -1) {
    return multiplier >= 0 && shift <= max_shift && shift >= -20;
}
// `fast` of a per-channel problem whose pairs all pass channel_pair_is_fast
inline int32_t channel_fast_mode(const eh_requant &q) {
    if (q.zp_out < -1024 || q.zp_out > 1024) return 0;
    return q.act_min >= q.zp_out ? 2 : 1;
}

// Four values in 0 .. 255 to the four bytes of a word, lowest first: two byte permutes and one OR
// (shift-and-OR takes four or five instructions).
__host__ __device__ __forceinline__ uint32_t pack_bytes(uint32_t b0, uint32_t b1, uint32_t b2, uint32_t b3) {
#if defined(__HIP_DEVICE_COMPILE__)
    // v_perm_b32(S0, S1, sel): selector bytes 0..3 pick from S1, 4..7 from S0, 0x0c gives zero
    return __builtin_amdgcn_perm(b1, b0, 0x0c0c0400u) | __builtin_amdgcn_perm(b3, b2, 0x04000c0cu);
#else
    return b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
#endif
}

// The first `cnt` (1 .. 16) of sixteen result bytes to a destination of any alignment: whole dwords at byte addresses
// (global memory takes them), single bytes for the last one to three.  The fallback of every epilogue whose rows do
// not start on 16-byte boundaries (an odd channel count) or end inside a 16-byte chunk.
typedef uint32_t u32_any_alignment __attribute__((aligned(1)));
__device__ __forceinline__ void store_bytes_any_alignment(uint8_t *dst, const uint32_t (&packed)[4], int cnt) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        if (cnt >= 4 * g + 4) {
            *reinterpret_cast<u32_any_alignment *>(dst + 4 * g) = packed[g];
        } else {
#pragma unroll
            for (int t = 0; t < 3; ++t)
                if (4 * g + t < cnt) dst[4 * g + t] = (uint8_t)(packed[g] >> (8 * t));
        }
    }
}

template <int MODE>
__host__ __device__ __forceinline__ uint32_t requant_u8_as(int32_t acc, const RequantDev &r) {
    if constexpr (MODE == 2)
        return requant_u8_fast_relu(acc, r);
    else if constexpr (MODE == 1)
        return requant_u8_fast(acc, r);
    else
        return requant_u8(acc, r);
}

inline RequantDev make_requant_dev(const eh_requant &q) {
    RequantDev r;
    r.multiplier = q.multiplier;
    r.left_shift = q.shift > 0 ? q.shift : 0;
    r.right_shift = q.shift > 0 ? 0 : -q.shift;
    r.mask = (int32_t)((1u << r.right_shift) - 1u);
    r.half = r.mask >> 1;
    r.zp_out = q.zp_out;
    r.act_min = q.act_min;
    r.act_max = q.act_max;
    // |xM| < 2^62 and the rounding term stays below 2^(42 + rs): no 64-bit overflow up to rs = 20
    r.fast = (r.left_shift == 0 && r.right_shift >= 1 && r.right_shift <= 20 && q.multiplier >= 0 && q.zp_out >= -1024 &&
              q.zp_out <= 1024)
                 ? 1
                 : 0;
    if (r.fast && q.act_min >= q.zp_out) r.fast = 2;
    r.fast_shift = r.fast ? r.right_shift - 1 : 0;
    const int rs = r.fast ? r.right_shift : 1;
    const int64_t pos = (1ll << 30) + (1ll << (30 + rs)) + (int64_t)q.zp_out * (1ll << (31 + rs));
    const int64_t neg = pos - (1ll << 31);
    r.pc_multiplier = nullptr;
    r.pc_shift = nullptr;
    r.lo_scaled = (int32_t)((uint32_t)q.act_min << r.fast_shift);
    r.hi_scaled = (int32_t)(((uint32_t)q.act_max << r.fast_shift) | ((1u << r.fast_shift) - 1u));
    r.pos_lo = (uint32_t)((uint64_t)pos & 0xFFFFFFFFull);
    r.pos_hi = (uint32_t)((uint64_t)pos >> 32);
    r.neg_lo = (uint32_t)((uint64_t)neg & 0xFFFFFFFFull);
    r.neg_hi = (uint32_t)((uint64_t)neg >> 32);
    return r;
}

// floor(n / d) for 0 <= n < 2^31 as (umulhi(mul, n) + n) >> shift
struct FastDiv {
    uint32_t mul = 1;
    uint32_t shift = 0;
};
inline FastDiv make_fastdiv(uint32_t d) {
    FastDiv f;
    uint32_t l = 0;
    while ((1ull << l) < d) ++l;
    f.shift = l;
    f.mul = (uint32_t)((((1ull << 32) * ((1ull << l) - d)) / d + 1) & 0xFFFFFFFFull);
    return f;
}
__device__ __forceinline__ uint32_t fastdiv(uint32_t n, const FastDiv &f) { return (__umulhi(f.mul, n) + n) >> f.shift; }

// signed_weights: zp_w is an int8 zero point; signed_io: zp_in, zp_out and the activation range are int8 values
int check_requant(const eh_requant *q, bool signed_weights = false, bool signed_io = false);

// ---------------------------------------------------------------- quantized add
// The reference's quantized add (gpu/operators/cl_kernels/AddKernelsQauntized.cpp:135-215): both inputs shifted
// left, brought to a common scale by a Q31 multiplier and a rounding right shift each, summed, rescaled, offset,
// clamped.  Lives here because the GEMM epilogues can apply it to their result and a residual tensor.
struct AddDev {
    int32_t zp_a, zp_b, zp_out, left_shift;
    int32_t mult_a, rs_a, mult_b, rs_b, mult_out, rs_out;
    int32_t act_min, act_max;
};

// SaturatingRoundingDoublingHighMul for a non-negative multiplier (no saturation case), then
// RoundingDivideByPOT
__host__ __device__ __forceinline__ int32_t mul_round_shift(int32_t x, int32_t mult, int32_t rs) {
    const int64_t ab = (int64_t)x * (int64_t)mult + (1ll << 30);
    const int32_t v = (int32_t)(ab >> 31);
    const int32_t mask = (int32_t)((1u << rs) - 1u);
    const int32_t rem = v & mask;
    const int32_t thr = (mask >> 1) - (v >> 31);
    return (v >> rs) + (rem > thr ? 1 : 0);
}

__host__ __device__ __forceinline__ uint32_t add_one(uint32_t a, uint32_t b, const AddDev &q) {
    const int32_t va = (int32_t)(((uint32_t)((int32_t)a - q.zp_a)) << q.left_shift);
    const int32_t vb = (int32_t)(((uint32_t)((int32_t)b - q.zp_b)) << q.left_shift);
    const int32_t sa = mul_round_shift(va, q.mult_a, q.rs_a);
    const int32_t sb = mul_round_shift(vb, q.mult_b, q.rs_b);
    int32_t r = mul_round_shift(sa + sb, q.mult_out, q.rs_out) + q.zp_out;
    r = r < q.act_min ? q.act_min : r;
    r = r > q.act_max ? q.act_max : r;
    return (uint32_t)r;
}

__host__ __device__ __forceinline__ uint32_t add_word(uint32_t a, uint32_t b, const AddDev &q) {
    return add_one(a & 255u, b & 255u, q) | (add_one((a >> 8) & 255u, (b >> 8) & 255u, q) << 8) |
           (add_one((a >> 16) & 255u, (b >> 16) & 255u, q) << 16) | (add_one(a >> 24, b >> 24, q) << 24);
}


inline AddDev make_add_dev(const eh_add_requant &q) {
    AddDev d;
    d.zp_a = q.zp_a;
    d.zp_b = q.zp_b;
    d.zp_out = q.zp_out;
    d.left_shift = q.left_shift;
    d.mult_a = q.mult_a;
    d.mult_b = q.mult_b;
    d.mult_out = q.mult_out;
    // a positive shift (a multiplier of 1 or more) is applied as no shift, as the reference kernel's fall-through does
    d.rs_a = q.shift_a < 0 ? -q.shift_a : 0;
    d.rs_b = q.shift_b < 0 ? -q.shift_b : 0;
    d.rs_out = q.shift_out < 0 ? -q.shift_out : 0;
    d.act_min = q.act_min;
    d.act_max = q.act_max;
    return d;
}
int check_add_requant(const eh_add_requant *q);
// out = add(a, b) over `count` bytes on `stream` (out may be a or b)
int launch_add_u8(const uint8_t *a, const uint8_t *b, uint8_t *out, int64_t count, const AddDev &d, hipStream_t stream);

// ---------------------------------------------------------------- implicit GEMM
// One row of the k-table describes one load unit (VEC bytes) of the reduction
// axis: where it sits relative to the top-left input pixel of an output pixel.
struct KUnit {
    int32_t offset;  // (dy * W + dx) * Cin + c, in bytes
    int16_t dy;
    int16_t dx;
};

// Kernel shape chosen for a problem when its weights are packed.
enum GemmConfigId {
    GEMM_STAGED = 0,            // register-staged kernel, any channel count; weights row-major [n_pad][k_pad]
    GEMM_DMA_256x128 = 1,       // direct-to-LDS kernels; weights in swizzled 1 KiB blocks (see packed_b_offset)
    GEMM_DMA_128x128 = 2,
    GEMM_DMA_128x64 = 3,
    GEMM_DMA_64x64_SPLITK = 4,
    GEMM_DMA_256x256 = 5,
    GEMM_THIN = 6,              // one-tap problems short of work for tiles; weights in MFMA fragment order
    GEMM_C3K3 = 7,              // 3 input channels, 3x3 taps (first layers); weights row-major [n_pad][32]
    GEMM_CONV3X3 = 8,           // 3x3 taps, stride 1, input patch staged in LDS once; weights in MFMA fragment order
    GEMM_SKINNY = 10,           // one tap, at most 64 output pixels, long reductions; weights in MFMA fragment order
    GEMM_ROWS = 9,              // 1 - 4 input channels, kernel rows of at most 32 bytes; weights row-major [n_pad][32 per kernel row]
};
struct GemmConfig {
    int32_t id = GEMM_STAGED;
    int32_t slab = 64;  // reduction bytes per stage; k_pad is a multiple of it
};

struct GemmProblem {
    const uint8_t *a;     // activations: NHWC image or [M][K] matrix
    const int8_t *b;      // packed weights, value = w - 128, laid out for cfg (see packed_b_offset)
    GemmConfig cfg;
    const uint8_t *fillbuf;  // 32 bytes: 16 x input zero point byte, then 16 x the byte that a_xor turns into 0
    const int32_t *bias;  // [n_pad] bias with the zero-point terms folded in
    const KUnit *ktab;    // [k_pad / vec]
    uint8_t *out;
    int32_t m, n;           // GEMM extents (n = output channels)
    int32_t k, k_pad;       // real and padded reduction length
    int32_t vec;            // bytes per load unit of A: 16, 4 or 1
    // input geometry: row m -> (img, oy, ox) over (ho, wo); top-left tap at
    // (oy * stride_h + y_base, ox * stride_w + x_base)
    int32_t h, w, cin;
    int32_t ho, wo;
    int32_t stride_h, stride_w, y_base, x_base;
    // output addressing: ((img * out_h + oy * out_sy + out_y0) * out_w + ox * out_sx + out_x0) * ldc + col
    int32_t out_h, out_w, out_sy, out_sx, out_y0, out_x0, ldc;
    FastDiv div_plane, div_wo;  // row decode: m / (ho * wo), rem / wo
    int32_t dense;     // 1: a plain [m][k] matrix with row stride cin and k a multiple of the slab (no taps, no padding)
    int32_t zw;        // zp_w - 128: coefficient of the per-row activation sum
    int32_t a_offset;  // one-tap problems: byte offset of the (group's) first channel within a pixel
    uint32_t fill;     // input zero point byte as it is stored, replicated in 4 bytes (value of an out-of-image tap)
    // int8 tensors (PrecisionType::INT8) run as their uint8 equivalents (value + 128, zero points + 128):
    uint32_t a_xor;    // turns four stored activation bytes into int8 MFMA operands: 0x80808080 for uint8 data, 0 for int8
    uint32_t out_xor;  // turns four uint8 results into the stored bytes: 0 for uint8 data, 0x80808080 for int8
    int32_t rows_kh, rows_kw;  // GEMM_ROWS: the kernel's extent (other kernels find their taps in ktab)
    // fused residual add (one-tap and split-reduction kernels only): out = add(residual, result) with `radd`;
    // `residual` is addressed like `out`.  Null: plain convolution.
    const uint8_t *residual;
    AddDev radd;
    RequantDev rq;
    // A slice of a reduction that several workgroups share (64 x 64 split-reduction tiles, table-driven): `ktab`, `b`
    // and `k_pad` describe the slice, `b_slabs` is the whole reduction's slab count (the distance between the packed
    // weights' row blocks; 0: k_pad / slab), and the tile's int32 sums minus its activation-sum term go to
    // partial[m * partial_ld + n] instead of being requantized (launch_splitk_finish adds the slices up and does that).
    int32_t *partial;
    int32_t partial_ld;
    int32_t b_slabs;
};

// Equally shaped problems of one operator that go out as one launch (kernel argument).
struct GemmBatch {
    static constexpr int MAX = 8;
    GemmProblem p[MAX];
};
int launch_igemm(const GemmProblem &p, hipStream_t stream);
// `count` problems in order; consecutive equally shaped ones that the direct-to-LDS kernels serve share launches
int launch_igemm_batch(const GemmProblem *ps, int count, hipStream_t stream);
int launch_igemm_dma(const GemmProblem *ps, int count, hipStream_t stream);  // vec == 16 and a k-table that fits LDS
GemmConfig igemm_dma_select(int32_t m, int32_t n, int32_t k, int32_t siblings);
inline size_t igemm_dma_ktab_limit() { return 12288; }
int launch_igemm_thin(const GemmProblem *ps, int count, hipStream_t stream);  // `count` equally shaped problems as one launch
// p: the whole problem (bias, requantization, output addressing, residual); partial: [slices][p.m][partial_ld] int32
int launch_splitk_finish(const GemmProblem &p, const int32_t *partial, int32_t partial_ld, int32_t slices, hipStream_t stream);
int launch_conv_c3k3(const GemmProblem &p, hipStream_t stream);
int launch_conv3x3_patch(const GemmProblem &p, hipStream_t stream);
// one tap, few output pixels, long reductions: cut along the weights (eh_gemm_skinny.hip)
bool gemm_skinny_applies(int32_t taps, int32_t cin_group, int32_t pixel_stride, int32_t channel_offset, int64_t m, int64_t n);
int launch_gemm_skinny(const GemmProblem &p, hipStream_t stream);
// few input channels, a kernel row per reduction step (eh_conv_rows.hip)
bool conv_rows_applies(int32_t cin_group, int32_t pixel_stride, int32_t kh, int32_t kw);
int launch_conv_rows(const GemmProblem &p, hipStream_t stream);
int conv3x3_patch_prepare();  // per device, from eh_init
bool conv3x3_patch_applies(int32_t cin_group, int32_t pixel_stride, int32_t wo, int32_t ho);
bool igemm_thin_applies(int32_t taps, int32_t cin_group, int32_t pixel_stride, int32_t channel_offset, int32_t y_base,
                        int32_t x_base, int64_t m, int64_t n);
// Byte offset of reduction chunk `kc16` (16-byte units) of packed weight row `n`.
// Direct-to-LDS layouts: 1 KiB blocks of (1024 / slab) rows x slab bytes, ordered
// [row block][slab index], the 16-byte chunks of a row XOR-swizzled by the row index.
// Within every block of 32 output channels the rows are permuted (channel
// 16h + 4g + t sits in row 8g + 4h + t): a lane of the 32x32x32 MFMA holds result
// rows 8g + 4h + t (h = lane / 32), which this way are 16 consecutive channels.
__host__ __device__ inline size_t packed_b_offset(const GemmConfig &cfg, int n, int kc16, int k_pad) {
    if (cfg.id == GEMM_STAGED || cfg.id == GEMM_C3K3 || cfg.id == GEMM_ROWS) return (size_t)n * k_pad + (size_t)kc16 * 16;
    const int ch = n & 31;
    n = (n & ~31) | (((ch & 15) >> 2) << 3) | ((ch >> 4) << 2) | (ch & 3);
    // fragment order: [32-channel block][32-byte step][lane = 32 * (chunk & 1) + row][16 bytes]
    if (cfg.id == GEMM_THIN || cfg.id == GEMM_CONV3X3 || cfg.id == GEMM_SKINNY) return ((((size_t)(n >> 5) * (k_pad / 32) + (kc16 >> 1)) * 2 + (kc16 & 1)) * 32 + (n & 31)) * 16;
    const int cpr = cfg.slab / 16, rpb = 1024 / cfg.slab;
    const int c = kc16 % cpr;
    return ((size_t)(n / rpb) * (k_pad / cfg.slab) + kc16 / cpr) * 1024 + (size_t)(n % rpb) * cfg.slab +
           ((c ^ (n & (cpr - 1))) << 4);
}
// tile extents the launcher will pick for (m, n): packed weights are padded to them
int igemm_n_tile(int32_t m, int32_t n, int32_t k);

// ---------------------------------------------------------------- packing
struct PackProblem {
    const uint8_t *w;      // source weights (uint8, or int8 when w_signed)
    int32_t w_signed;      // the bytes are int8 values (per-channel quantized weights): packed as they are, not minus 128
    const int32_t *bias;   // source bias [n] or null
    int8_t *b;             // [n_pad][k_pad]
    int32_t *colsum;       // [n_pad]  sum_k (w - 128)
    GemmConfig cfg;
    int32_t n, n_pad, cin, taps, k, k_pad;
    int32_t row_bytes;     // GEMM_ROWS: kw * cin, the bytes of a kernel row, which starts every 32 packed bytes; else 0
    int32_t cin_real;      // channels the source weights hold per tap when `cin` counts padding channels behind them (those pack as 0); 0 = cin
    // source index of (out channel o, in channel c, tap t) = o*so + c*sc + tap_off[t]
    int64_t so, sc;
    // n_period != 0: packed row o is output channel o % n_period of the (o / n_period)-th of several kernel columns
    // that share a launch, and its source index is (o % n_period)*so + (o / n_period)*period_step + c*sc + tap_off[t]
    int32_t n_period;
    int64_t period_step;
    // block_cin != 0: several convolution groups as one block-diagonal problem.  Packed row o belongs to group
    // o / block_n of the bundle and reduction channel c to group c / block_cin; where the two differ the row holds
    // `off_block` (the weight zero point minus 128, so that the product with any activation is zero), elsewhere
    // source channel c % block_cin.
    int32_t block_cin, block_n, off_block;
    const int32_t *tap_off;  // device [taps]
};
int launch_pack_weights(const PackProblem &p, hipStream_t stream);
// folded[n] = bias[n] - za * colsum[n] + k * za * zw   (za = zp_in - 128, zw = zp_w - 128); bias_period != 0: bias[n % bias_period]
// also refreshes the 32-byte fill constant when `fillbuf` is not null
int launch_fold_bias(const int32_t *bias, const int32_t *colsum, int32_t *folded, int32_t n, int32_t n_pad,
                     int32_t k, int32_t zp_in, int32_t zp_w, uint8_t *fillbuf, int32_t io_flip, hipStream_t stream, int32_t bias_period = 0);

// ---------------------------------------------------------------- depthwise
struct DwProblem {
    const uint8_t *in;
    const uint8_t *w;            // raw weights [cout][kh*kw] (uint8, or int8 bytes when w_signed)
    const int32_t *bias;         // raw bias [cout] or null
    const int32_t *w_pair;       // [ceil(taps/2)][cout]: (w[2p]-zp_w) | (w[2p+1]-zp_w) << 16 as int16 halves
    const int32_t *bias_folded;  // [cout]: bias - zp_in * sum_t (w - zp_w)
    // 3x3 weights whose differences w - zp_w all fit int8 (else null): [3 columns][cout] words holding a column's
    // three vertical taps in bytes 0..2, and the bias with (zp_in - 128) * sum_t (w - zp_w) folded in
    const int32_t *w_trip;
    const int32_t *bias_trip;
    // 3x3 weights of any range for the unsigned dot product form (else null): [3 columns][cout] words of the uint8
    // weight bytes (int8 weights: byte + 128), and the bias with -zp_in * sum w + 9 zp_in zp_w folded in
    const int32_t *w_fold;
    const int32_t *bias_fold;
    // 5x5 and 7x7 weights of any range for the same form (else null): [kw columns][2][cout] words of a column's
    // vertical taps 0..3 and 4..kh-1 as uint8 bytes, and the bias with -zp_in * sum w + kh kw zp_in zp_w folded in
    const int32_t *w_foldk;
    const int32_t *bias_foldk;
    uint8_t *out;
    int32_t n, c, h, w_, cout, dm;
    int32_t kh, kw, stride_h, stride_w, pad_t, pad_l, dil_h, dil_w;
    int32_t ho, wo;
    int32_t zp_in, zp_w;
    int32_t w_signed;            // weight bytes are int8
    uint32_t io_flip;            // 0x80808080 when input and output hold int8 values (computed as value + 128), else 0
    RequantDev rq;               // rq.pc_multiplier / rq.pc_shift: [cout + 4] when set
};
int launch_dw_pack(const uint8_t *w, const int32_t *bias, int32_t *w_pair, int32_t *bias_folded, int32_t cout,
                   int32_t taps, int32_t zp_in, int32_t zp_w, int32_t w_signed, hipStream_t stream);
int launch_dw_pack_trip(const uint8_t *w, const int32_t *bias, int32_t *w_trip, int32_t *bias_trip, int32_t cout, int32_t zp_in,
                        int32_t zp_w, int32_t w_signed, hipStream_t stream);
int launch_dw_pack_fold(const uint8_t *w, const int32_t *bias, int32_t *w_fold, int32_t *bias_fold, int32_t cout, int32_t zp_in,
                        int32_t zp_w_u8, int32_t w_signed, hipStream_t stream);
int launch_dw_pack_foldk(const uint8_t *w, const int32_t *bias, int32_t *w_foldk, int32_t *bias_foldk, int32_t cout, int32_t k,
                         int32_t zp_in, int32_t zp_w_u8, int32_t w_signed, hipStream_t stream);
int launch_dwconv_nhwc(const DwProblem &p, hipStream_t stream);
int launch_dwconv_nchw(const DwProblem &p, hipStream_t stream);

// ---------------------------------------------------------------- pointwise + depthwise in one launch (eh_block.hip)
bool pwdw_block_applies(const GemmProblem &pw, const DwProblem &dw);
bool pwdw_block_listed(int32_t images, int32_t image_h, int32_t image_w, int32_t in_channels, int32_t expanded_channels, int32_t stride);
bool pwdw_block_preferred(const GemmProblem &pw, const DwProblem &dw);  // the fused launch is the faster one for this shape (measured table)
int launch_pwdw_block(const GemmProblem &pw, const DwProblem &dw, int rows_per_tile, int cols_per_tile, hipStream_t stream);

// ---------------------------------------------------------------- layout
int launch_nchw2nhwc(const uint8_t *src, uint8_t *dst, int32_t n, int32_t c, int32_t hw, hipStream_t stream);
// dst[pixel][c * times + d] = src[pixel][c] for d < times; rows of c_to >= c * times bytes (a multiple of 4), the tail
// filled with repeats of the pixel's last channel
int launch_replicate_channels(const uint8_t *src, uint8_t *dst, int64_t pixels, int32_t c, int32_t times, int32_t c_to, hipStream_t stream);
// dst[pixel][0 .. c_keep) = src[pixel][0 .. c_keep) from rows of c_from bytes (a multiple of 4)
int launch_keep_channels(const uint8_t *src, uint8_t *dst, int64_t pixels, int32_t c_from, int32_t c_keep, hipStream_t stream);
// dst[pixel][g][0 .. cg_to) = src[pixel][g][0 .. cg) followed by cg_to - cg bytes `fill`, for `groups` channel groups per pixel
int launch_pad_channels(const uint8_t *src, uint8_t *dst, int64_t pixels, int32_t groups, int32_t cg, int32_t cg_to, uint32_t fill,
                        hipStream_t stream);
int launch_nhwc2nchw(const uint8_t *src, uint8_t *dst, int32_t n, int32_t c, int32_t hw, hipStream_t stream);

}  // namespace eh
