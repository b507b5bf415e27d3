// Weight packing, bias folding and layout conversion kernels (gfx950).
//
// Packing stands in for the reference's weight repack kernels
// (alignQuantizedWeight_gemm, gpu/operators/cl_kernels/ConvolutionKernels.cpp:1276-1315;
// align_weight_direct and update_direct_conv_bias,
// DirectConvolutionKernel.cpp:4289-4322,4871-4884; matrixTrans/weightAlign,
// DeconvolutionKernels.cpp:8-22,269-282).  Layout conversion stands in for
// nchw2nhwc_uint8 / nhwc2nchw_uint8 (gpu/common/CLKernels.hpp:429-491).
#include "eh_internal.h"

namespace eh {
namespace {

// One workgroup per packed row (output channel): writes w - 128 as int8 in the
// reduction order (tap, channel), zero beyond the real extents, and the row sum.
__global__ __launch_bounds__(256) void pack_weights_kernel(const PackProblem p) {
    __shared__ int32_t partial[256];
    const int o = blockIdx.x;
    int32_t sum = 0;
    for (int k = threadIdx.x; k < p.k_pad; k += 256) {
        int32_t v = 0;
        // source position in (tap, channel) order: k itself, or with one kernel row per 32 packed bytes, row * row_bytes + byte
        const int kk = p.row_bytes ? ((k & 31) < p.row_bytes ? (k >> 5) * p.row_bytes + (k & 31) : p.k) : k;
        if (o < p.n && kk < p.k) {
            const int t = kk / p.cin, c = kk - t * p.cin;
            if (p.block_cin) {
                if (c / p.block_cin == o / p.block_n) {
                    const uint8_t raw = p.w[(int64_t)o * p.so + (int64_t)(c % p.block_cin) * p.sc + p.tap_off[t]];
                    v = p.w_signed ? (int32_t)(int8_t)raw : (int32_t)raw - 128;
                } else {
                    v = p.off_block;
                }
            } else if (p.cin_real == 0 || c < p.cin_real) {
                const int64_t row = p.n_period ? (int64_t)(o % p.n_period) * p.so + (int64_t)(o / p.n_period) * p.period_step : (int64_t)o * p.so;
                const uint8_t raw = p.w[row + (int64_t)c * p.sc + p.tap_off[t]];
                v = p.w_signed ? (int32_t)(int8_t)raw : (int32_t)raw - 128;
            }
        }
        p.b[packed_b_offset(p.cfg, o, k >> 4, p.k_pad) + (k & 15)] = (int8_t)v;
        sum += v;
    }
    partial[threadIdx.x] = sum;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) partial[threadIdx.x] += partial[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) p.colsum[o] = partial[0];
}

__global__ void fold_bias_kernel(const int32_t *bias, const int32_t *colsum, int32_t *folded, int32_t n, int32_t n_pad,
                                 int32_t k, int32_t za, int32_t zw, uint8_t *fillbuf, int32_t io_flip, int32_t bias_period) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    // bytes as the input tensor stores them: int8 tensors (io_flip = 0x80) hold value - 128
    if (fillbuf && i < 32) fillbuf[i] = (uint8_t)((i < 16 ? za + 128 : 0x80) ^ io_flip);
    if (i >= n_pad) return;
    int32_t v = 0;
    if (i < n) v = (bias ? bias[bias_period ? i % bias_period : i] : 0) - za * colsum[i] + k * za * zw;
    folded[i] = v;
}

// Channel padding: rows of `cg` bytes (a pixel's channels, or one group's) copied to rows of `cg_to` bytes, the tail set
// to `fill`.  Stands in for the reference's pad-and-align passes over activations (PadConvertKernels.cpp:25-167 pads the
// reduction length of the im2col matrix to a multiple of 16).  One thread per destination dword; source dwords
// are read at byte addresses.
typedef uint32_t u32_a1 __attribute__((aligned(1)));
__global__ __launch_bounds__(256) void pad_channels_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, const uint32_t total,
                                                           const FastDiv div_quads, const int32_t cg, const int32_t cg_to, const uint32_t fill) {
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    if (idx >= total) return;
    const uint32_t row = fastdiv(idx, div_quads), quad = idx - row * (uint32_t)(cg_to >> 2);
    const int c = (int)quad * 4;
    const uint8_t *s = src + ((size_t)row * (size_t)cg + (size_t)c);
    uint32_t v;
    if (c + 4 <= cg) {
        v = *reinterpret_cast<const u32_a1 *>(s);
    } else {
        v = fill * 0x01010101u;
        for (int b = 0; c + b < cg; ++b) v = (v & ~(0xFFu << (8 * b))) | ((uint32_t)s[b] << (8 * b));
    }
    reinterpret_cast<uint32_t *>(dst)[idx] = v;
}

// Every channel `times` times in a row: what a depthwise convolution with a depth multiplier reads, laid out so that
// output channel j reads input channel j of the copy (DepthwiseconvolutionKernels.cpp:1242-1321 indexes the input by
// out_channel / depth_multiplier instead).  One thread per destination dword.
__global__ __launch_bounds__(256) void replicate_channels_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, const uint32_t total,
                                                                 const uint32_t quads_per_pixel, const FastDiv div_quads, const int32_t c,
                                                                 const FastDiv div_times) {
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    if (idx >= total) return;
    const uint32_t pixel = fastdiv(idx, div_quads), quad = idx - pixel * quads_per_pixel;
    const uint8_t *s = src + (size_t)pixel * (size_t)c;
    uint32_t v = 0;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        const uint32_t ch = fastdiv(quad * 4u + (uint32_t)b, div_times);  // (past the last channel in a row's padding tail)
        v |= (uint32_t)s[ch < (uint32_t)c ? ch : (uint32_t)c - 1u] << (8 * b);
    }
    reinterpret_cast<uint32_t *>(dst)[idx] = v;
}

// The first c_keep bytes of every row of c_from bytes: the caller's channels out of an image computed on a channel count
// rounded up to a multiple of 4.  One thread per source dword; whole dwords leave at byte addresses.
__global__ __launch_bounds__(256) void keep_channels_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, const uint32_t total,
                                                            const uint32_t quads_per_pixel, const FastDiv div_quads, const int32_t c_keep) {
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    if (idx >= total) return;
    const uint32_t pixel = fastdiv(idx, div_quads), quad = idx - pixel * quads_per_pixel;
    const uint32_t v = reinterpret_cast<const uint32_t *>(src)[idx];
    const int left = c_keep - (int)quad * 4;
    uint8_t *d = dst + ((size_t)pixel * (size_t)c_keep + (size_t)quad * 4u);
    if (left >= 4) {
        *reinterpret_cast<u32_a1 *>(d) = v;
    } else {
        for (int b = 0; b < left; ++b) d[b] = (uint8_t)(v >> (8 * b));
    }
}

// Byte-matrix transpose per batch: src [batch][R][S] -> dst [batch][S][R].
// 64x64 tiles through LDS; 4-byte global accesses when the extents allow.
constexpr int TT = 64;
__global__ __launch_bounds__(256) void transpose_u8_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                           int32_t R, int32_t S) {
    __shared__ __align__(4) uint8_t tile[TT][TT + 4];
    const size_t batch_off = (size_t)blockIdx.z * R * S;
    src += batch_off;
    dst += batch_off;
    const int r0 = blockIdx.y * TT, s0 = blockIdx.x * TT;
    const int t = threadIdx.x;
    const bool src_wide = (S & 3) == 0 && (reinterpret_cast<uintptr_t>(src) & 3) == 0;
    const bool dst_wide = (R & 3) == 0 && (reinterpret_cast<uintptr_t>(dst) & 3) == 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = (t >> 4) + 16 * i, s4 = (t & 15) * 4;
        const int gr = r0 + r, gs = s0 + s4;
        uint32_t v = 0;
        if (gr < R) {
            if (src_wide && gs + 4 <= S) {
                v = *reinterpret_cast<const uint32_t *>(src + (size_t)gr * S + gs);
            } else {
                for (int b = 0; b < 4; ++b)
                    if (gs + b < S) v |= (uint32_t)src[(size_t)gr * S + gs + b] << (8 * b);
            }
        }
        *reinterpret_cast<uint32_t *>(&tile[r][s4]) = v;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int s = (t >> 4) + 16 * i, r4 = (t & 15) * 4;
        const int gs = s0 + s, gr = r0 + r4;
        if (gs >= S || gr >= R) continue;
        const uint32_t v = (uint32_t)tile[r4][s] | ((uint32_t)tile[r4 + 1][s] << 8) | ((uint32_t)tile[r4 + 2][s] << 16) |
                           ((uint32_t)tile[r4 + 3][s] << 24);
        if (dst_wide && gr + 4 <= R) {
            *reinterpret_cast<uint32_t *>(dst + (size_t)gs * R + gr) = v;
        } else {
            for (int b = 0; b < 4; ++b)
                if (gr + b < R) dst[(size_t)gs * R + gr + b] = (uint8_t)(v >> (8 * b));
        }
    }
}

// The same transpose for extents that are multiples of 4 on both axes (most feature maps): 16 KiB tiles of
// TR rows x TS columns, 16-byte global loads along S and 16-byte global stores along R, so a wave instruction
// moves whole 128-byte lines on either side when the extents are multiples of 16 (other multiples of 4 take
// the same accesses at dword boundaries and finish rows and row groups with single dwords).  A thread brings four 16-byte chunks into LDS, then gathers a
// block of 16 rows x 4 columns as sixteen dwords, transposes its four 4x4 byte blocks in registers (two
// rounds of byte permutes) and stores, for each of its four columns, sixteen consecutive row bytes.
// Three tile shapes: 128x128, 32x512 for few rows (NCHW -> NHWC with up to 32 channels) and 512x32 for few
// columns (the way back).  The 16-byte chunks of an LDS row are XOR-swizzled by the 16-row group (the rows
// themselves in the 32-column shape), which makes the dword gathers of a half wave fall on 32 distinct banks.
__device__ __forceinline__ void transpose4x4_bytes(const uint32_t a0, const uint32_t a1, const uint32_t a2, const uint32_t a3,
                                                   uint32_t out[4]) {
    const uint32_t lo01 = __builtin_amdgcn_perm(a1, a0, 0x05010400u), hi01 = __builtin_amdgcn_perm(a1, a0, 0x07030602u);
    const uint32_t lo23 = __builtin_amdgcn_perm(a3, a2, 0x05010400u), hi23 = __builtin_amdgcn_perm(a3, a2, 0x07030602u);
    out[0] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
    out[1] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
    out[2] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
    out[3] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
}

// four dwords at a 4-byte aligned address (global memory takes a dwordx4 access at any dword boundary)
typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));

template <int TR, int TS>
__global__ __launch_bounds__(256) void transpose_u8_wide_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                                int32_t R, int32_t S) {
    static_assert(TR * TS == 16384 && TR % 16 == 0 && TS % 16 == 0, "a 16 KiB tile, four chunks per thread");
    constexpr int CPR = TS / 16;   // 16-byte chunks per tile row
    constexpr int NRG = TR / 16;   // 16-row groups per tile
    __shared__ __align__(16) uint8_t tile[TR * TS];
    // where chunk c of row r sits in LDS
    auto lds_pos = [](int r, int c) -> int {
        if constexpr (TS == 32)
            return ((r ^ ((r >> 4) & 3)) * CPR + c) * 16;
        else if constexpr (NRG >= 8)
            return (r * CPR + (c ^ ((r >> 4) & (CPR - 1)))) * 16;
        else
            return (r * CPR + (c ^ ((r >> 4) * (8 / NRG)))) * 16;
    };
    const size_t batch_off = (size_t)blockIdx.z * R * S;
    src += batch_off;
    dst += batch_off;
    const int r0 = blockIdx.y * TR, s0 = blockIdx.x * TS;
    const int t = threadIdx.x;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int idx = t + 256 * it, row = idx / CPR, c = idx % CPR;
        const int gr = r0 + row, gs = s0 + 16 * c;
        if (gr < R && gs < S) {
            const uint8_t *g = src + (size_t)gr * S + gs;
            u32x4_a4 v = {0u, 0u, 0u, 0u};
            if (gs + 16 <= S) {
                v = *reinterpret_cast<const u32x4_a4 *>(g);
            } else {  // the last chunk of a row whose length is a multiple of 4 only
#pragma unroll
                for (int d = 0; d < 4; ++d)
                    if (gs + 4 * d < S) v[d] = *reinterpret_cast<const uint32_t *>(g + 4 * d);
            }
            *reinterpret_cast<uint4 *>(tile + lds_pos(row, c)) = make_uint4(v[0], v[1], v[2], v[3]);
        }
    }
    __syncthreads();
    // this thread's block: rows 16*rg .. 16*rg+15, columns 4*cg .. 4*cg+3
    int rg, cg;
    if constexpr (TS == 32) {
        cg = t & 7;
        rg = t >> 3;
    } else {
        rg = t % NRG;
        cg = t / NRG;
    }
    const int gr = r0 + 16 * rg;
    if (gr >= R) return;
    uint32_t col[4][4];  // [column][row quad]
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        uint32_t a[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) a[i] = *reinterpret_cast<const uint32_t *>(tile + lds_pos(16 * rg + 4 * q + i, cg >> 2) + (cg & 3) * 4);
        uint32_t o[4];
        transpose4x4_bytes(a[0], a[1], a[2], a[3], o);
#pragma unroll
        for (int k = 0; k < 4; ++k) col[k][q] = o[k];
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int gs = s0 + 4 * cg + k;
        if (gs >= S) continue;
        uint8_t *g = dst + (size_t)gs * R + gr;
        if (gr + 16 <= R) {
            const u32x4_a4 v = {col[k][0], col[k][1], col[k][2], col[k][3]};
            *reinterpret_cast<u32x4_a4 *>(g) = v;
        } else {
#pragma unroll
            for (int q = 0; q < 4; ++q)
                if (gr + 4 * q < R) *reinterpret_cast<uint32_t *>(g + 4 * q) = col[k][q];
        }
    }
}

// Two to four rows (an RGB image's planes to interleaved pixels) or two to four columns (the way back), the long
// extent a multiple of 4: a thread moves four positions of the long axis, one dword per plane on the planar side and
// C consecutive dwords on the interleaved side, so both sides are whole, coalesced dword accesses.  (The tiled kernels
// would leave nine tenths of a tile empty.)
template <int C, bool INTERLEAVE>
__global__ __launch_bounds__(256) void transpose_u8_few_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, int32_t L) {
    const int i = blockIdx.x * 256 + threadIdx.x;  // positions 4 i .. 4 i + 3 of the long axis
    if (4 * i >= L) return;
    const size_t batch_off = (size_t)blockIdx.z * C * L;
    const uint8_t *plane_side = (INTERLEAVE ? src : dst) + batch_off + 4 * (size_t)i;
    const uint8_t *pixel_side = (INTERLEAVE ? dst : src) + batch_off + 4 * (size_t)i * C;
    uint32_t planes[C], pixels[C];
    if constexpr (INTERLEAVE) {
#pragma unroll
        for (int c = 0; c < C; ++c) planes[c] = *reinterpret_cast<const uint32_t *>(plane_side + (size_t)c * L);
#pragma unroll
        for (int d = 0; d < C; ++d) pixels[d] = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int c = 0; c < C; ++c) pixels[(j * C + c) >> 2] |= ((planes[c] >> (8 * j)) & 255u) << (8 * ((j * C + c) & 3));
#pragma unroll
        for (int d = 0; d < C; ++d) *reinterpret_cast<uint32_t *>(const_cast<uint8_t *>(pixel_side) + 4 * d) = pixels[d];
    } else {
#pragma unroll
        for (int d = 0; d < C; ++d) pixels[d] = *reinterpret_cast<const uint32_t *>(pixel_side + 4 * d);
#pragma unroll
        for (int c = 0; c < C; ++c) planes[c] = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int c = 0; c < C; ++c) planes[c] |= ((pixels[(j * C + c) >> 2] >> (8 * ((j * C + c) & 3))) & 255u) << (8 * j);
#pragma unroll
        for (int c = 0; c < C; ++c) *reinterpret_cast<uint32_t *>(const_cast<uint8_t *>(plane_side) + (size_t)c * L) = planes[c];
    }
}

template <bool INTERLEAVE>
int launch_transpose_few(const uint8_t *src, uint8_t *dst, int32_t batch, int32_t c, int32_t L, hipStream_t stream) {
    const dim3 grid((unsigned)((L / 4 + 255) / 256), 1, (unsigned)batch);
    if (c == 2)
        hipLaunchKernelGGL((transpose_u8_few_kernel<2, INTERLEAVE>), grid, dim3(256), 0, stream, src, dst, L);
    else if (c == 3)
        hipLaunchKernelGGL((transpose_u8_few_kernel<3, INTERLEAVE>), grid, dim3(256), 0, stream, src, dst, L);
    else
        hipLaunchKernelGGL((transpose_u8_few_kernel<4, INTERLEAVE>), grid, dim3(256), 0, stream, src, dst, L);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

int launch_transpose(const uint8_t *src, uint8_t *dst, int32_t batch, int32_t R, int32_t S, hipStream_t stream) {
    if (batch <= 0 || R <= 0 || S <= 0) return EH_OK;
    EH_REQUIRE(batch <= 65535, "transpose: batch %d exceeds the grid limit", batch);
    const bool dwords = ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 3) == 0;
    if (dwords && R >= 2 && R <= 4 && S % 4 == 0 && S >= 64) return launch_transpose_few<true>(src, dst, batch, R, S, stream);
    if (dwords && S >= 2 && S <= 4 && R % 4 == 0 && R >= 64) return launch_transpose_few<false>(src, dst, batch, S, R, stream);
    if (R % 4 == 0 && S % 4 == 0 && ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 3) == 0) {
        if (S <= 32 && (R + 511) / 512 <= 65535) {
            hipLaunchKernelGGL((transpose_u8_wide_kernel<512, 32>), dim3(1, (R + 511) / 512, batch), dim3(256), 0, stream, src, dst, R, S);
            EH_HIP(hipGetLastError());
            return EH_OK;
        }
        if (R <= 32) {
            hipLaunchKernelGGL((transpose_u8_wide_kernel<32, 512>), dim3((S + 511) / 512, 1, batch), dim3(256), 0, stream, src, dst, R, S);
            EH_HIP(hipGetLastError());
            return EH_OK;
        }
        if ((R + 127) / 128 <= 65535) {
            hipLaunchKernelGGL((transpose_u8_wide_kernel<128, 128>), dim3((S + 127) / 128, (R + 127) / 128, batch), dim3(256), 0, stream, src, dst, R, S);
            EH_HIP(hipGetLastError());
            return EH_OK;
        }
    }
    const dim3 grid((S + TT - 1) / TT, (R + TT - 1) / TT, batch);
    hipLaunchKernelGGL(transpose_u8_kernel, grid, dim3(256), 0, stream, src, dst, R, S);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

}  // namespace

int launch_replicate_channels(const uint8_t *src, uint8_t *dst, int64_t pixels, int32_t c, int32_t times, int32_t c_to, hipStream_t stream) {
    EH_REQUIRE(c > 0 && times > 0 && c_to >= c * times && (c_to & 3) == 0, "replicate_channels: bad extents %d x %d -> %d", c, times, c_to);
    const int64_t total = pixels * (c_to >> 2);
    if (total <= 0) return EH_OK;
    EH_REQUIRE(total < (1ll << 31), "replicate_channels: tensor too large");
    hipLaunchKernelGGL(replicate_channels_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, src, dst, (uint32_t)total,
                       (uint32_t)(c_to >> 2), make_fastdiv((uint32_t)(c_to >> 2)), c, make_fastdiv((uint32_t)times));
    EH_HIP(hipGetLastError());
    return EH_OK;
}

int launch_keep_channels(const uint8_t *src, uint8_t *dst, int64_t pixels, int32_t c_from, int32_t c_keep, hipStream_t stream) {
    EH_REQUIRE(c_keep > 0 && c_from >= c_keep && (c_from & 3) == 0, "keep_channels: bad extents %d of %d", c_keep, c_from);
    const int64_t total = pixels * (c_from >> 2);
    if (total <= 0) return EH_OK;
    EH_REQUIRE(total < (1ll << 31), "keep_channels: tensor too large");
    hipLaunchKernelGGL(keep_channels_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, src, dst, (uint32_t)total,
                       (uint32_t)(c_from >> 2), make_fastdiv((uint32_t)(c_from >> 2)), c_keep);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

int launch_pad_channels(const uint8_t *src, uint8_t *dst, int64_t pixels, int32_t groups, int32_t cg, int32_t cg_to, uint32_t fill,
                        hipStream_t stream) {
    EH_REQUIRE(groups > 0 && cg > 0 && cg_to >= cg && (cg_to & 3) == 0, "pad_channels: bad extents %d x %d -> %d", groups, cg, cg_to);
    const int64_t total = pixels * groups * (cg_to >> 2);
    if (total <= 0) return EH_OK;
    EH_REQUIRE(total < (1ll << 31) && pixels * groups * cg < (1ll << 31), "pad_channels: tensor too large");
    hipLaunchKernelGGL(pad_channels_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, src, dst, (uint32_t)total,
                       make_fastdiv((uint32_t)(cg_to >> 2)), cg, cg_to, fill & 0xFFu);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

int launch_pack_weights(const PackProblem &p, hipStream_t stream) {
    if (p.n_pad <= 0) return EH_OK;
    hipLaunchKernelGGL(pack_weights_kernel, dim3(p.n_pad), dim3(256), 0, stream, p);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

int launch_fold_bias(const int32_t *bias, const int32_t *colsum, int32_t *folded, int32_t n, int32_t n_pad, int32_t k,
                     int32_t zp_in, int32_t zp_w, uint8_t *fillbuf, int32_t io_flip, hipStream_t stream, int32_t bias_period) {
    if (n_pad <= 0) return EH_OK;
    hipLaunchKernelGGL(fold_bias_kernel, dim3((n_pad + 255) / 256), dim3(256), 0, stream, bias, colsum, folded, n, n_pad,
                       k, zp_in - 128, zp_w - 128, fillbuf, io_flip, bias_period);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

// out[n][hw][c] = in[n][c][hw]
int launch_nchw2nhwc(const uint8_t *src, uint8_t *dst, int32_t n, int32_t c, int32_t hw, hipStream_t stream) {
    return launch_transpose(src, dst, n, c, hw, stream);
}

// out[n][c][hw] = in[n][hw][c]
int launch_nhwc2nchw(const uint8_t *src, uint8_t *dst, int32_t n, int32_t c, int32_t hw, hipStream_t stream) {
    return launch_transpose(src, dst, n, hw, c, stream);
}

}  // namespace eh
