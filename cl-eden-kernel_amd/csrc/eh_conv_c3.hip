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
//
// With 32 output channels or more the multiply-adds go to the matrix cores instead (conv_c3k3_mfma_kernel): a
// lane still gathers one pixel, the two halves of the wave then exchange half of what they gathered so that each
// of the wave's two 32-pixel blocks has its 27 (+5 zero) reduction bytes in 32x32x32 fragment form, and one
// v_mfma_i32_32x32x32_i8 per block and 32 channels leaves every lane with 16 consecutive channels of one pixel.
//
// Stands in for the reference's direct convolution kernels on this shape
// (gpu/operators/cl_kernels/DirectConvolutionKernel.cpp, 3x3 uint8 variants).
#include <type_traits>

#include "eh_internal.h"

namespace eh {
namespace {

typedef uint32_t u32_unaligned __attribute__((aligned(1)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));

// The 27 reduction bytes of output pixel m as seven dwords of a' = a ^ a_xor (the 28th byte zero), out-of-image taps
// reading the input zero point; all zero for m past the last pixel.
__device__ __forceinline__ void gather_c3k3(const GemmProblem &p, const uint32_t in_bytes, int m, uint32_t (&A)[7]) {
    const int plane = p.ho * p.wo;
    const int img = (int)fastdiv((uint32_t)m, p.div_plane), rem = m - img * plane;
    const int oy = (int)fastdiv((uint32_t)rem, p.div_wo), ox = rem - oy * p.wo;
    const int iy0 = oy * p.stride_h + p.y_base, ix0 = ox * p.stride_w + p.x_base;
    const bool c0 = (unsigned)ix0 < (unsigned)p.w, c1 = (unsigned)(ix0 + 1) < (unsigned)p.w, c2 = (unsigned)(ix0 + 2) < (unsigned)p.w;
    const int row_bytes = p.w * 3, a_row0 = ((img * p.h + iy0) * p.w + ix0) * 3;
    uint32_t seg[3][3];  // per kernel row: bytes 0..8 = 3 pixels x 3 channels, the rest zero
#pragma unroll
    for (int ky = 0; ky < 3; ++ky) {
        const int iy = iy0 + ky;
        const bool row_ok = (unsigned)iy < (unsigned)p.h;
        // (tensors stay below 2 GiB: 32-bit offsets, one multiplication chain per pixel instead of one per row)
        const int a = a_row0 + ky * row_bytes;
        uint32_t d0 = 0, d1 = 0, d2 = 0;
        if (row_ok) {
            if (a >= 0 && (uint32_t)a + 12u <= in_bytes) {
                d0 = *reinterpret_cast<const u32_unaligned *>(p.a + a);
                d1 = *reinterpret_cast<const u32_unaligned *>(p.a + a + 4);
                d2 = *reinterpret_cast<const u32_unaligned *>(p.a + a + 8);
            } else {  // the first pixel of the first image and the last of the last: byte by byte, inside the tensor
                for (int j = 0; j < 9; ++j) {
                    const int b = a + j;
                    const uint32_t v = b >= 0 && (uint32_t)b < in_bytes ? p.a[b] : 0u;
                    if (j < 4) d0 |= v << (8 * j);
                    else if (j < 8) d1 |= v << (8 * (j - 4));
                    else d2 |= v;
                }
            }
        }
        const bool v0 = row_ok && c0, v1 = row_ok && c1, v2 = row_ok && c2;
        const uint32_t m0 = (v0 ? 0x00FFFFFFu : 0u) | (v1 ? 0xFF000000u : 0u);
        const uint32_t m1 = (v1 ? 0x0000FFFFu : 0u) | (v2 ? 0xFFFF0000u : 0u);
        const uint32_t m2 = v2 ? 0x000000FFu : 0u;
        seg[ky][0] = (d0 & m0) | (p.fill & ~m0);
        seg[ky][1] = (d1 & m1) | (p.fill & ~m1);
        seg[ky][2] = ((d2 & m2) | (p.fill & ~m2)) & 0xFFu;
    }
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
    if (m >= p.m) {
#pragma unroll
        for (int i = 0; i < 7; ++i) A[i] = 0;
    }
}

// Matrix-core form.  Grid: x = 256 pixels per workgroup (64 per wave).  With one multiplier and shift per channel,
// FAST means that every channel's pair is inside the single-shift form's range.
template <bool ROWSUM, bool FAST>
__global__ __launch_bounds__(256) void conv_c3k3_mfma_kernel(const GemmProblem p, const uint32_t in_bytes) {
    const int lane = threadIdx.x & 63, r = lane & 31, half = lane >> 5;
    // every XCD (workgroups are dispatched round-robin over the 8 of them) takes one contiguous eighth of the
    // pixel range, so the input rows that neighbouring output rows share are fetched into one L2 only
    const int block = (int)((blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3));
    const int m_own = block * 256 + threadIdx.x;  // the pixel this lane gathers
    uint32_t A[7];
    gather_c3k3(p, in_bytes, m_own < p.m ? m_own : p.m - 1, A);
    if (m_own >= p.m) {
#pragma unroll
        for (int i = 0; i < 7; ++i) A[i] = 0;
    }
    int rs_own = 0;
    if constexpr (ROWSUM) {
#pragma unroll
        for (int i = 0; i < 7; ++i) rs_own = __builtin_amdgcn_sdot4((int)A[i], 0x01010101, rs_own, false);
    }
    // Lanes 0..31 hold pixels 0..31 of the wave, lanes 32..63 pixels 32..63.  Block b's fragment wants, in lane
    // (r, half), reduction bytes 16 half .. 16 half + 15 of pixel 32 b + r: the lower lanes send the upper half of
    // their bytes up (block 0), the upper lanes send the lower half of theirs down (block 1).
    uint32_t got[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) got[d] = (uint32_t)__shfl_xor((int)(half ? A[d] : (d < 3 ? A[4 + d] : 0u)), 32);
    v4i af[2];
    af[0] = half ? v4i{(int)got[0], (int)got[1], (int)got[2], (int)got[3]} : v4i{(int)A[0], (int)A[1], (int)A[2], (int)A[3]};
    af[1] = half ? v4i{(int)A[4], (int)A[5], (int)A[6], 0} : v4i{(int)got[0], (int)got[1], (int)got[2], (int)got[3]};
    const int rs_got = ROWSUM ? __shfl_xor(rs_own, 32) : 0;
    const int wave_base = m_own - lane;
    const RequantDev rq = p.rq;
    const int plane = p.ho * p.wo;
    const int n_blocks = (p.n + 31) >> 5;
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        const int m = wave_base + 32 * b + r;  // the pixel whose 16 channels this lane finishes in block b
        const int ncorr = ROWSUM ? -p.zw * (b == half ? rs_own : rs_got) : 0;
        size_t out_off = 0;
        if (m < p.m) {
            const int img = (int)fastdiv((uint32_t)m, p.div_plane), rem = m - img * plane;
            const int oy = (int)fastdiv((uint32_t)rem, p.div_wo), ox = rem - oy * p.wo;
            out_off = (((size_t)img * p.out_h + (oy * p.out_sy + p.out_y0)) * p.out_w + (ox * p.out_sx + p.out_x0)) * (size_t)p.ldc;
        }
        for (int nb = 0; nb < n_blocks; ++nb) {
            // weight rows are stored plainly, [channel][32 bytes]: row `r` of the fragment is channel 16 h + 4 g + t of the block
            const int ch = nb * 32 + 16 * ((r >> 2) & 1) + 4 * (r >> 3) + (r & 3);
            const v4i wf = *reinterpret_cast<const v4i *>(p.b + (size_t)ch * 32 + half * 16);
            const int n = nb * 32 + half * 16;
            // the accumulators start from the folded bias and the pixel's row-sum term: nothing left to add afterwards
            v16i acc;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int4 bb = *reinterpret_cast<const int4 *>(p.bias + n + g * 4);
                acc[g * 4 + 0] = bb.x + ncorr;
                acc[g * 4 + 1] = bb.y + ncorr;
                acc[g * 4 + 2] = bb.z + ncorr;
                acc[g * 4 + 3] = bb.w + ncorr;
            }
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf, af[b], acc, 0, 0, 0);
            uint32_t packed[4];
            auto produce = [&](auto mode_c) {
                constexpr int mode = decltype(mode_c)::value;
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    if (rq.pc_multiplier) {  // (the arrays are padded past the last channel block)
                        const int4 cm = *reinterpret_cast<const int4 *>(rq.pc_multiplier + n + g * 4);
                        const int4 cs = *reinterpret_cast<const int4 *>(rq.pc_shift + n + g * 4);
                        auto one = [&](int x, int32_t mult, int32_t shift) {
                            if constexpr (mode == 0)
                                return requant_u8_channel(x, mult, shift, rq);
                            else
                                return requant_u8_channel_fast<mode>(x, mult, shift, rq);
                        };
                        packed[g] = pack_bytes(one(acc[g * 4 + 0], cm.x, cs.x), one(acc[g * 4 + 1], cm.y, cs.y),
                                               one(acc[g * 4 + 2], cm.z, cs.z), one(acc[g * 4 + 3], cm.w, cs.w)) ^
                                    p.out_xor;
                        continue;
                    }
                    if constexpr (mode != 0)
                        packed[g] = requant4_fast<mode>(acc[g * 4 + 0], acc[g * 4 + 1], acc[g * 4 + 2], acc[g * 4 + 3], 0, rq) ^ p.out_xor;
                    else
                        packed[g] = pack_bytes(requant_u8_as<mode>(acc[g * 4 + 0], rq), requant_u8_as<mode>(acc[g * 4 + 1], rq),
                                               requant_u8_as<mode>(acc[g * 4 + 2], rq), requant_u8_as<mode>(acc[g * 4 + 3], rq)) ^
                                    p.out_xor;
                }
            };
            if constexpr (!FAST)
                produce(std::integral_constant<int, 0>{});
            else if (rq.fast == 2)
                produce(std::integral_constant<int, 2>{});
            else
                produce(std::integral_constant<int, 1>{});
            if (m < p.m && n < p.n) {
                uint8_t *dst = p.out + out_off + n;
                const int cnt = p.n - n;
                if (cnt >= 16 && (p.ldc & 3) == 0 && (reinterpret_cast<uintptr_t>(p.out) & 3) == 0) {
                    *reinterpret_cast<u32x4_a4 *>(dst) = u32x4_a4{packed[0], packed[1], packed[2], packed[3]};
                } else {
                    store_bytes_any_alignment(dst, packed, cnt < 16 ? cnt : 16);
                }
            }
        }
    }
}

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
        packed[g] = pack_bytes(o[0], o[1], o[2], o[3]) ^ p.out_xor;
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
        store_bytes_any_alignment(dst, packed, p.n - n0 < 16 ? p.n - n0 : 16);
    }
}

}  // namespace

int launch_conv_c3k3(const GemmProblem &p, hipStream_t stream) {
    EH_REQUIRE(p.k == 27 && p.k_pad == 32 && p.cin == 3, "conv_c3k3: not a 3-channel 3x3 problem");
    const size_t in_bytes = (size_t)p.h * p.w * 3;  // per image
    const int images = (p.m + p.ho * p.wo - 1) / (p.ho * p.wo);
    EH_REQUIRE(in_bytes * images < (1ull << 31), "conv_c3k3: input too large");
    const uint32_t total_bytes = (uint32_t)(in_bytes * images);
    const bool rowsum = p.zw != 0;
    bool fast = p.rq.fast != 0;
    if (p.n >= 32) {  // the packed rows and the folded bias are padded to whole tiles of channels
        const dim3 grid_m(((p.m + 255) / 256 + 7) / 8 * 8);  // whole multiples of 8: see the kernel's block numbering
        if (rowsum && fast)
            hipLaunchKernelGGL((conv_c3k3_mfma_kernel<true, true>), grid_m, dim3(256), 0, stream, p, total_bytes);
        else if (rowsum)
            hipLaunchKernelGGL((conv_c3k3_mfma_kernel<true, false>), grid_m, dim3(256), 0, stream, p, total_bytes);
        else if (fast)
            hipLaunchKernelGGL((conv_c3k3_mfma_kernel<false, true>), grid_m, dim3(256), 0, stream, p, total_bytes);
        else
            hipLaunchKernelGGL((conv_c3k3_mfma_kernel<false, false>), grid_m, dim3(256), 0, stream, p, total_bytes);
        EH_HIP(hipGetLastError());
        return EH_OK;
    }
    const dim3 grid((p.m + 255) / 256, (p.n + 15) / 16);
    if (p.rq.pc_multiplier) fast = false;  // this kernel's per-channel code is the two-step order
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
