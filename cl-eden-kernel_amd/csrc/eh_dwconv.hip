// Depthwise uint8 convolution (gfx950): bandwidth-bound, no matrix cores.
//
// Replaces the reference's depthwise kernels for the uint8 path
// (gpu/operators/cl_kernels/DepthwiseconvolutionKernels.cpp:1242-2290: generic
// depthwise_conv plus the 3x3 pad-merge specialisations) and their pad pass
// (PadConvertKernels.cpp:7-23).  Out-of-image taps read the input zero point,
// as the reference's padding does, so they contribute nothing.
//
// Channels-last fast path: one thread owns four adjacent channels of one output
// pixel, so a wavefront reads whole contiguous pixel rows.  Two taps of one
// channel are paired into a 16-bit dot product (v_dot2_i32_i16) against
// weights stored as (w - zp_w) int16 pairs; the input zero point is folded
// into the bias: sum (a - zi)(w - zw) = sum a (w - zw) - zi * sum (w - zw).
#include "eh_internal.h"

namespace eh {
namespace {

typedef short v2s __attribute__((ext_vector_type(2)));

__device__ __forceinline__ int dot2(uint32_t a_pair, int32_t w_pair, int acc) {
    return __builtin_amdgcn_sdot2(__builtin_bit_cast(v2s, a_pair), __builtin_bit_cast(v2s, w_pair), acc, false);
}

// byte j of `lo` into bits 0..15 and byte j of `hi` into bits 16..31, zero extended
template <int J>
__device__ __forceinline__ uint32_t pair_bytes(uint32_t lo, uint32_t hi) {
    constexpr uint32_t sel = (0x0cu << 24) | ((4u + J) << 16) | (0x0cu << 8) | (uint32_t)J;
    return __builtin_amdgcn_perm(hi, lo, sel);
}

template <int KH, int KW>
__global__ __launch_bounds__(256) void dw_nhwc_vec4_kernel(const DwProblem p, const long total) {
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int cq_count = p.c >> 2;
    const int cq = (int)(idx % cq_count);
    const long pix = idx / cq_count;
    const int ox = (int)(pix % p.wo);
    const long t0 = pix / p.wo;
    const int oy = (int)(t0 % p.ho), img = (int)(t0 / p.ho);
    const int kh = KH ? KH : p.kh, kw = KW ? KW : p.kw;
    const int taps = kh * kw, pairs = (taps + 1) >> 1;
    const int iy0 = oy * p.stride_h - p.pad_t, ix0 = ox * p.stride_w - p.pad_l;
    const uint8_t *src = p.in + (size_t)img * p.h * p.w_ * p.c + cq * 4;
    const uint32_t fill = (uint32_t)p.zp_in * 0x01010101u;

    auto tap = [&](int t) -> uint32_t {
        if (t >= taps) return 0u;
        const int ky = t / kw, kx = t - ky * kw;
        const int iy = iy0 + ky * p.dil_h, ix = ix0 + kx * p.dil_w;
        if ((unsigned)iy < (unsigned)p.h && (unsigned)ix < (unsigned)p.w_)
            return *reinterpret_cast<const uint32_t *>(src + ((size_t)iy * p.w_ + ix) * p.c);
        return fill;
    };

    const int4 b4 = *reinterpret_cast<const int4 *>(p.bias_folded + cq * 4);
    int acc0 = b4.x, acc1 = b4.y, acc2 = b4.z, acc3 = b4.w;
#pragma unroll
    for (int pr = 0; pr < (KH ? (KH * KW + 1) / 2 : 1); ++pr) {
        if constexpr (KH == 0) break;
        const uint32_t lo = tap(2 * pr), hi = tap(2 * pr + 1);
        const int4 w4 = *reinterpret_cast<const int4 *>(p.w_pair + (size_t)pr * p.cout + cq * 4);
        acc0 = dot2(pair_bytes<0>(lo, hi), w4.x, acc0);
        acc1 = dot2(pair_bytes<1>(lo, hi), w4.y, acc1);
        acc2 = dot2(pair_bytes<2>(lo, hi), w4.z, acc2);
        acc3 = dot2(pair_bytes<3>(lo, hi), w4.w, acc3);
    }
    if constexpr (KH == 0) {
        for (int pr = 0; pr < pairs; ++pr) {
            const uint32_t lo = tap(2 * pr), hi = tap(2 * pr + 1);
            const int4 w4 = *reinterpret_cast<const int4 *>(p.w_pair + (size_t)pr * p.cout + cq * 4);
            acc0 = dot2(pair_bytes<0>(lo, hi), w4.x, acc0);
            acc1 = dot2(pair_bytes<1>(lo, hi), w4.y, acc1);
            acc2 = dot2(pair_bytes<2>(lo, hi), w4.z, acc2);
            acc3 = dot2(pair_bytes<3>(lo, hi), w4.w, acc3);
        }
    }
    uint32_t o;
    if (p.rq.fast)
        o = requant_u8_fast(acc0, p.rq) | (requant_u8_fast(acc1, p.rq) << 8) | (requant_u8_fast(acc2, p.rq) << 16) |
            (requant_u8_fast(acc3, p.rq) << 24);
    else
        o = requant_u8(acc0, p.rq) | (requant_u8(acc1, p.rq) << 8) | (requant_u8(acc2, p.rq) << 16) |
            (requant_u8(acc3, p.rq) << 24);
    *reinterpret_cast<uint32_t *>(p.out + (size_t)pix * p.cout + cq * 4) = o;
}

// One output element per thread; any depth multiplier, dilation, channel count.
// NHWC = true: channel fastest.  NHWC = false: planar NCHW, x fastest.
template <bool NHWC>
__global__ __launch_bounds__(256) void dw_scalar_kernel(const DwProblem p, const long total) {
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    int oc, ox, oy, img;
    if (NHWC) {
        oc = (int)(idx % p.cout);
        long r = idx / p.cout;
        ox = (int)(r % p.wo);
        r /= p.wo;
        oy = (int)(r % p.ho);
        img = (int)(r / p.ho);
    } else {
        ox = (int)(idx % p.wo);
        long r = idx / p.wo;
        oy = (int)(r % p.ho);
        r /= p.ho;
        oc = (int)(r % p.cout);
        img = (int)(r / p.cout);
    }
    const int ic = oc / p.dm;
    int32_t acc = p.bias ? p.bias[oc] : 0;
    const int iy0 = oy * p.stride_h - p.pad_t, ix0 = ox * p.stride_w - p.pad_l;
    for (int ky = 0; ky < p.kh; ++ky) {
        const int iy = iy0 + ky * p.dil_h;
        if ((unsigned)iy >= (unsigned)p.h) continue;
        for (int kx = 0; kx < p.kw; ++kx) {
            const int ix = ix0 + kx * p.dil_w;
            if ((unsigned)ix >= (unsigned)p.w_) continue;
            const size_t a_idx = NHWC ? (((size_t)img * p.h + iy) * p.w_ + ix) * p.c + ic
                                      : (((size_t)img * p.c + ic) * p.h + iy) * p.w_ + ix;
            const int32_t a = (int32_t)p.in[a_idx] - p.zp_in;
            const int32_t w = (int32_t)p.w[((size_t)oc * p.kh + ky) * p.kw + kx] - p.zp_w;
            acc += a * w;
        }
    }
    p.out[idx] = (uint8_t)requant_u8(acc, p.rq);
}

__global__ void dw_pack_kernel(const uint8_t *w, const int32_t *bias, int32_t *w_pair, int32_t *bias_folded, int32_t cout,
                               int32_t taps, int32_t zp_in, int32_t zp_w) {
    const int oc = blockIdx.x * blockDim.x + threadIdx.x;
    if (oc >= cout) return;
    int32_t sum = 0;
    const int pairs = (taps + 1) >> 1;
    for (int pr = 0; pr < pairs; ++pr) {
        const int32_t lo = (int32_t)w[(size_t)oc * taps + 2 * pr] - zp_w;
        const int32_t hi = 2 * pr + 1 < taps ? (int32_t)w[(size_t)oc * taps + 2 * pr + 1] - zp_w : 0;
        sum += lo + hi;
        w_pair[(size_t)pr * cout + oc] = (int32_t)(((uint32_t)lo & 0xFFFFu) | ((uint32_t)hi << 16));
    }
    bias_folded[oc] = (bias ? bias[oc] : 0) - zp_in * sum;
}

}  // namespace

int launch_dw_pack(const uint8_t *w, const int32_t *bias, int32_t *w_pair, int32_t *bias_folded, int32_t cout,
                   int32_t taps, int32_t zp_in, int32_t zp_w, hipStream_t stream) {
    if (cout <= 0) return EH_OK;
    hipLaunchKernelGGL(dw_pack_kernel, dim3((cout + 127) / 128), dim3(128), 0, stream, w, bias, w_pair, bias_folded, cout,
                       taps, zp_in, zp_w);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

int launch_dwconv_nhwc(const DwProblem &p, hipStream_t stream) {
    const long outs = (long)p.n * p.ho * p.wo * p.cout;
    if (outs <= 0) return EH_OK;
    const bool vec = p.dm == 1 && (p.c & 3) == 0 && (reinterpret_cast<uintptr_t>(p.in) & 3) == 0 &&
                     (reinterpret_cast<uintptr_t>(p.out) & 3) == 0;
    if (vec) {
        const long total = outs / 4;
        const long blocks = (total + 255) / 256;
        EH_REQUIRE(blocks < (1l << 31), "depthwise: grid too large");
        if (p.kh == 3 && p.kw == 3)
            hipLaunchKernelGGL((dw_nhwc_vec4_kernel<3, 3>), dim3((unsigned)blocks), dim3(256), 0, stream, p, total);
        else
            hipLaunchKernelGGL((dw_nhwc_vec4_kernel<0, 0>), dim3((unsigned)blocks), dim3(256), 0, stream, p, total);
    } else {
        const long blocks = (outs + 255) / 256;
        EH_REQUIRE(blocks < (1l << 31), "depthwise: grid too large");
        hipLaunchKernelGGL((dw_scalar_kernel<true>), dim3((unsigned)blocks), dim3(256), 0, stream, p, outs);
    }
    EH_HIP(hipGetLastError());
    return EH_OK;
}

int launch_dwconv_nchw(const DwProblem &p, hipStream_t stream) {
    const long outs = (long)p.n * p.ho * p.wo * p.cout;
    if (outs <= 0) return EH_OK;
    const long blocks = (outs + 255) / 256;
    EH_REQUIRE(blocks < (1l << 31), "depthwise: grid too large");
    hipLaunchKernelGGL((dw_scalar_kernel<false>), dim3((unsigned)blocks), dim3(256), 0, stream, p, outs);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

}  // namespace eh
