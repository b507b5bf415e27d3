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
        if (o < p.n && k < p.k) {
            const int t = k / p.cin, c = k - t * p.cin;
            const uint8_t raw = p.w[(int64_t)o * p.so + (int64_t)c * p.sc + p.tap_off[t]];
            v = p.w_signed ? (int32_t)(int8_t)raw : (int32_t)raw - 128;
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
                                 int32_t k, int32_t za, int32_t zw, uint8_t *fillbuf, int32_t io_flip) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    // bytes as the input tensor stores them: int8 tensors (io_flip = 0x80) hold value - 128
    if (fillbuf && i < 32) fillbuf[i] = (uint8_t)((i < 16 ? za + 128 : 0x80) ^ io_flip);
    if (i >= n_pad) return;
    int32_t v = 0;
    if (i < n) v = (bias ? bias[i] : 0) - za * colsum[i] + k * za * zw;
    folded[i] = v;
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

int launch_transpose(const uint8_t *src, uint8_t *dst, int32_t batch, int32_t R, int32_t S, hipStream_t stream) {
    if (batch <= 0 || R <= 0 || S <= 0) return EH_OK;
    EH_REQUIRE(batch <= 65535, "transpose: batch %d exceeds the grid limit", batch);
    const dim3 grid((S + TT - 1) / TT, (R + TT - 1) / TT, batch);
    hipLaunchKernelGGL(transpose_u8_kernel, grid, dim3(256), 0, stream, src, dst, R, S);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

}  // namespace

int launch_pack_weights(const PackProblem &p, hipStream_t stream) {
    if (p.n_pad <= 0) return EH_OK;
    hipLaunchKernelGGL(pack_weights_kernel, dim3(p.n_pad), dim3(256), 0, stream, p);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

int launch_fold_bias(const int32_t *bias, const int32_t *colsum, int32_t *folded, int32_t n, int32_t n_pad, int32_t k,
                     int32_t zp_in, int32_t zp_w, uint8_t *fillbuf, int32_t io_flip, hipStream_t stream) {
    if (n_pad <= 0) return EH_OK;
    hipLaunchKernelGGL(fold_bias_kernel, dim3((n_pad + 255) / 256), dim3(256), 0, stream, bias, colsum, folded, n, n_pad,
                       k, zp_in - 128, zp_w - 128, fillbuf, io_flip);
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
