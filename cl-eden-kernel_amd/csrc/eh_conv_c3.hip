// First-layer convolution: 3 input channels, 3x3 taps (any stride and padding),
// channels-last uint8.  The 27 reduction bytes of an output pixel are three runs
// of nine contiguous input bytes (one per kernel row), so no im2col staging is
// needed: a thread gathers them with three unaligned 12-byte reads, replaces the
// taps that fall outside the image by the input zero point, and holds them as
// seven signed dwords.  It then produces 16 output channels with v_dot4 against
// weight rows that are uniform across the wave (scalar loads), requantizes and
// writes 16 bytes.  Arithmetic is the implicit-GEMM one: a' = a ^ 0x80 against
// w - 128 with the zero-point terms folded into the bias and a per-pixel
// correction -(zp_w - 128) * sum(a').
//
// Stands in for the reference's direct convolution kernels on this shape
// (gpu/operators/cl_kernels/DirectConvolutionKernel.cpp, 3x3 uint8 variants).
#include <type_traits>

#include "eh_internal.h"

namespace eh {
namespace {

typedef uint32_t u32_unaligned __attribute__((aligned(1)));

template <bool ROWSUM, bool FAST>
__global__ __launch_bounds__(256) void conv_c3k3_kernel(const GemmProblem p, const uint32_t in_bytes) {
    const int m = blockIdx.x * 256 + threadIdx.x;
    if (m >= p.m) return;
    const int n0 = blockIdx.y * 16;
    const int plane = p.ho * p.wo;
    const int img = (int)fastdiv((uint32_t)m, p.div_plane), rem = m - img * plane;
    const int oy = (int)fastdiv((uint32_t)rem, p.div_wo), ox = rem - oy * p.wo;
    const int iy0 = oy * p.stride_h + p.y_base, ix0 = ox * p.stride_w + p.x_base;
    const bool c0 = (unsigned)ix0 < (unsigned)p.w, c1 = (unsigned)(ix0 + 1) < (unsigned)p.w, c2 = (unsigned)(ix0 + 2) < (unsigned)p.w;

    uint32_t seg[3][3];  // per kernel row: bytes 0..8 = 3 pixels x 3 channels, the rest zero
#pragma unroll
    for (int ky = 0; ky < 3; ++ky) {
        const int iy = iy0 + ky;
        const bool row_ok = (unsigned)iy < (unsigned)p.h;
        const long a = ((long)(img * p.h + iy) * p.w + ix0) * 3;
        uint32_t d0 = 0, d1 = 0, d2 = 0;
        if (row_ok) {
            if (a >= 0 && a + 12 <= (long)in_bytes) {
                d0 = *reinterpret_cast<const u32_unaligned *>(p.a + a);
                d1 = *reinterpret_cast<const u32_unaligned *>(p.a + a + 4);
                d2 = *reinterpret_cast<const u32_unaligned *>(p.a + a + 8);
            } else {  // the first pixel of the first image and the last of the last: byte by byte, inside the tensor
                for (int j = 0; j < 9; ++j) {
                    const long b = a + j;
                    const uint32_t v = b >= 0 && b < (long)in_bytes ? p.a[b] : 0u;
                    if (j < 4) d0 |= v << (8 * j);
                    else if (j < 8) d1 |= v << (8 * (j - 4));
                    else d2 |= v;
                }
            }
        }
        // keep the bytes of pixels inside the image, the others read the input zero point
        const bool v0 = row_ok && c0, v1 = row_ok && c1, v2 = row_ok && c2;
        const uint32_t m0 = (v0 ? 0x00FFFFFFu : 0u) | (v1 ? 0xFF000000u : 0u);
        const uint32_t m1 = (v1 ? 0x0000FFFFu : 0u) | (v2 ? 0xFFFF0000u : 0u);
        const uint32_t m2 = v2 ? 0x000000FFu : 0u;
        seg[ky][0] = (d0 & m0) | (p.fill & ~m0);
        seg[ky][1] = (d1 & m1) | (p.fill & ~m1);
        seg[ky][2] = ((d2 & m2) | (p.fill & ~m2)) & 0xFFu;
    }
    // reduction order (kernel row, kernel column, channel): 27 bytes in seven dwords, the 28th byte is zero
    uint32_t A[7];
    A[0] = seg[0][0];
    A[1] = seg[0][1];
    A[2] = seg[0][2] | (seg[1][0] << 8);
    A[3] = __builtin_amdgcn_alignbyte(seg[1][1], seg[1][0], 3);
    A[4] = (__builtin_amdgcn_alignbyte(seg[1][2], seg[1][1], 3) & 0xFFFFu) | (seg[2][0] << 16);
    A[5] = __builtin_amdgcn_alignbyte(seg[2][1], seg[2][0], 2);
    A[6] = __builtin_amdgcn_alignbyte(seg[2][2], seg[2][1], 2);
#pragma unroll
    for (int i = 0; i < 7; ++i) A[i] ^= p.a_xor;
    A[6] &= 0x00FFFFFFu;
    int ncorr = 0;
    if constexpr (ROWSUM) {
        int rs = 0;
#pragma unroll
        for (int i = 0; i < 7; ++i) rs = __builtin_amdgcn_sdot4((int)A[i], 0x01010101, rs, false);
        ncorr = -p.zw * rs;
    }
    const RequantDev rq = p.rq;
    uint32_t packed[4];
    auto produce = [&](auto mode_c) {
    constexpr int mode = decltype(mode_c)::value;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        uint32_t o[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int n = n0 + g * 4 + t;  // uniform across the wave: the weight row and bias come through the scalar unit
            const int *wrow = reinterpret_cast<const int *>(p.b + (size_t)n * 32);
            int acc = p.bias[n] + ncorr;
#pragma unroll
            for (int i = 0; i < 7; ++i) acc = __builtin_amdgcn_sdot4((int)A[i], wrow[i], acc, false);
            o[t] = mode == 0 && rq.pc_multiplier ? requant_u8_channel(acc, rq.pc_multiplier[n], rq.pc_shift[n], rq)
                                                 : requant_u8_as<mode>(acc, rq);
        }
        packed[g] = (o[0] | (o[1] << 8) | (o[2] << 16) | (o[3] << 24)) ^ p.out_xor;
    }
    };
    if constexpr (!FAST)
        produce(std::integral_constant<int, 0>{});
    else if (rq.fast == 2)
        produce(std::integral_constant<int, 2>{});
    else
        produce(std::integral_constant<int, 1>{});
    uint8_t *dst = p.out + (((size_t)img * p.out_h + (oy * p.out_sy + p.out_y0)) * p.out_w + (ox * p.out_sx + p.out_x0)) * (size_t)p.ldc + n0;
    const bool aligned16 = (p.ldc & 15) == 0 && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
    if (aligned16 && n0 + 16 <= p.n) {
        *reinterpret_cast<uint4 *>(dst) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
    } else {
        const int cnt = p.n - n0 < 16 ? p.n - n0 : 16;
        for (int t = 0; t < cnt; ++t) dst[t] = (uint8_t)(packed[t >> 2] >> (8 * (t & 3)));
    }
}

}  // namespace

int launch_conv_c3k3(const GemmProblem &p, hipStream_t stream) {
    EH_REQUIRE(p.k == 27 && p.k_pad == 32 && p.cin == 3, "conv_c3k3: not a 3-channel 3x3 problem");
    const size_t in_bytes = (size_t)p.h * p.w * 3;  // per image
    const int images = (p.m + p.ho * p.wo - 1) / (p.ho * p.wo);
    EH_REQUIRE(in_bytes * images < (1ull << 31), "conv_c3k3: input too large");
    const uint32_t total_bytes = (uint32_t)(in_bytes * images);
    const dim3 grid((p.m + 255) / 256, (p.n + 15) / 16);
    const bool rowsum = p.zw != 0, fast = p.rq.fast != 0;
    if (rowsum && fast)
        hipLaunchKernelGGL((conv_c3k3_kernel<true, true>), grid, dim3(256), 0, stream, p, total_bytes);
    else if (rowsum)
        hipLaunchKernelGGL((conv_c3k3_kernel<true, false>), grid, dim3(256), 0, stream, p, total_bytes);
    else if (fast)
        hipLaunchKernelGGL((conv_c3k3_kernel<false, true>), grid, dim3(256), 0, stream, p, total_bytes);
    else
        hipLaunchKernelGGL((conv_c3k3_kernel<false, false>), grid, dim3(256), 0, stream, p, total_bytes);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

}  // namespace eh
