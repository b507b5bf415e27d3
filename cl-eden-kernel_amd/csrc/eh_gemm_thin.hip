// uint8 GEMM kernel for 1x1 convolutions and fully-connected layers whose
// reduction length is at most 64 bytes (pointwise expansions such as 24 -> 144).
//
// Such layers move far more bytes than they multiply, so nothing is staged in
// LDS: a wave owns 32 output pixels, every lane fetches its 16 reduction bytes of
// its pixel straight into the 32x32x32 MFMA fragment layout (a row of K <= 64
// bytes is one or two such fragments; the bytes of a wave are one contiguous
// span when the pixels are), and the weights, packed in fragment order, are read
// per 32-channel block as one coalesced 1 KiB wave load that stays in L2.
// The weight fragment is the row operand and its rows are permuted within a
// 32-channel block (see packed_b_offset), so a lane ends up with 16 consecutive
// output channels of its pixel: requantize, pack, one 16-byte store.
#include "eh_internal.h"

namespace eh {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

namespace {

template <int KSTEPS, bool ROWSUM, bool FAST>
__global__ __launch_bounds__(256) void thin_gemm_kernel(const GemmProblem p, const int n_blocks) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 31, half = lane >> 5;
    const int m = (blockIdx.x * 4 + wave) * 32 + r;
    const bool row_ok = m < p.m;
    const int plane = p.ho * p.wo;

    // this lane's pixel: where its reduction bytes start, where its outputs go
    size_t in_off = 0, out_off = 0;
    if (row_ok) {
        const int img = (int)fastdiv((uint32_t)m, p.div_plane), rem = m - img * plane;
        const int oy = (int)fastdiv((uint32_t)rem, p.div_wo), ox = rem - oy * p.wo;
        in_off = ((size_t)(img * p.h + oy * p.stride_h + p.y_base) * p.w + (ox * p.stride_w + p.x_base)) * (size_t)p.cin +
                 (size_t)p.ktab[0].offset;
        out_off = (((size_t)img * p.out_h + (oy * p.out_sy + p.out_y0)) * p.out_w + (ox * p.out_sx + p.out_x0)) * (size_t)p.ldc;
    }
    // reduction bytes past K read as 0x80, which the signed shift turns into 0
    v4i af[KSTEPS];
    int rowsum = 0;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
        const int kb = ks * 32 + half * 16;
        uint2 lo = make_uint2(0x80808080u, 0x80808080u), hi = lo;
        if (row_ok && kb < p.k) lo = *reinterpret_cast<const uint2 *>(p.a + in_off + kb);
        if (row_ok && kb + 8 < p.k) hi = *reinterpret_cast<const uint2 *>(p.a + in_off + kb + 8);
        af[ks].x = (int)(lo.x ^ 0x80808080u);
        af[ks].y = (int)(lo.y ^ 0x80808080u);
        af[ks].z = (int)(hi.x ^ 0x80808080u);
        af[ks].w = (int)(hi.y ^ 0x80808080u);
        if constexpr (ROWSUM) {
            rowsum = __builtin_amdgcn_sdot4(af[ks].x, 0x01010101, rowsum, false);
            rowsum = __builtin_amdgcn_sdot4(af[ks].y, 0x01010101, rowsum, false);
            rowsum = __builtin_amdgcn_sdot4(af[ks].z, 0x01010101, rowsum, false);
            rowsum = __builtin_amdgcn_sdot4(af[ks].w, 0x01010101, rowsum, false);
        }
    }
    int ncorr = 0;
    if constexpr (ROWSUM) {
        rowsum += __shfl_xor(rowsum, 32);  // the other half of this pixel's reduction bytes
        ncorr = -p.zw * rowsum;
    }
    const RequantDev rq = p.rq;
    const bool aligned16 = (p.ldc & 15) == 0 && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
    const v4i *bfrag = reinterpret_cast<const v4i *>(p.b) + lane;

    // four channel blocks at a time: all their weight fragments and bias values are requested
    // before the first is used, so one memory latency covers the group
    // (blockIdx.y splits the channel blocks between workgroups when there are few pixels)
    constexpr int NBU = 4;
    for (int nb0 = blockIdx.y * NBU; nb0 < n_blocks; nb0 += gridDim.y * NBU) {
        v4i bf[NBU][KSTEPS];
        int4 bb[NBU][4];
#pragma unroll
        for (int u = 0; u < NBU; ++u) {
            const int nb = nb0 + u < n_blocks ? nb0 + u : n_blocks - 1;
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) bf[u][ks] = bfrag[(nb * KSTEPS + ks) * 64];
#pragma unroll
            for (int g = 0; g < 4; ++g) bb[u][g] = *reinterpret_cast<const int4 *>(p.bias + nb * 32 + half * 16 + g * 4);
        }
#pragma unroll
        for (int u = 0; u < NBU; ++u) {
            const int nb = nb0 + u;
            if (nb >= n_blocks) break;
            v16i acc;
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[i] = 0;
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[u][ks], af[ks], acc, 0, 0, 0);
            const int n = nb * 32 + half * 16;  // this lane's 16 consecutive channels
            uint32_t packed[4];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const uint32_t o0 = requant_u8_as<FAST>(acc[g * 4 + 0] + bb[u][g].x + ncorr, rq);
                const uint32_t o1 = requant_u8_as<FAST>(acc[g * 4 + 1] + bb[u][g].y + ncorr, rq);
                const uint32_t o2 = requant_u8_as<FAST>(acc[g * 4 + 2] + bb[u][g].z + ncorr, rq);
                const uint32_t o3 = requant_u8_as<FAST>(acc[g * 4 + 3] + bb[u][g].w + ncorr, rq);
                packed[g] = o0 | (o1 << 8) | (o2 << 16) | (o3 << 24);
            }
            if (!row_ok || n >= p.n) continue;
            uint8_t *dst = p.out + out_off + n;
            if (aligned16 && n + 16 <= p.n) {
                *reinterpret_cast<uint4 *>(dst) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
            } else {
                const int cnt = p.n - n < 16 ? p.n - n : 16;
                for (int t = 0; t < cnt; ++t) dst[t] = (uint8_t)(packed[t >> 2] >> (8 * (t & 3)));
            }
        }
    }
}

template <int KSTEPS>
int launch_steps(const GemmProblem &p, hipStream_t stream) {
    const int n_blocks = (p.n + 31) / 32;
    // enough waves to fill 256 CUs several times over: with few pixels the channel blocks are spread over grid.y too
    const int row_groups = (p.m + 127) / 128, n_groups = (n_blocks + 3) / 4;
    int split = 1;
    while (split < n_groups && (long)row_groups * split < 2048) ++split;
    const dim3 grid(row_groups, split);
    if (p.zw != 0) {
        if (p.rq.fast)
            hipLaunchKernelGGL((thin_gemm_kernel<KSTEPS, true, true>), grid, dim3(256), 0, stream, p, n_blocks);
        else
            hipLaunchKernelGGL((thin_gemm_kernel<KSTEPS, true, false>), grid, dim3(256), 0, stream, p, n_blocks);
    } else {
        if (p.rq.fast)
            hipLaunchKernelGGL((thin_gemm_kernel<KSTEPS, false, true>), grid, dim3(256), 0, stream, p, n_blocks);
        else
            hipLaunchKernelGGL((thin_gemm_kernel<KSTEPS, false, false>), grid, dim3(256), 0, stream, p, n_blocks);
    }
    EH_HIP(hipGetLastError());
    return EH_OK;
}

}  // namespace

// A single tap at the pixel itself (1x1 kernel, no padding), rows of at most 64
// reduction bytes that start on 8-byte boundaries.
bool igemm_thin_applies(int32_t taps, int32_t cin_group, int32_t pixel_stride, int32_t channel_offset, int32_t y_base,
                        int32_t x_base) {
    return taps == 1 && y_base == 0 && x_base == 0 && cin_group > 0 && cin_group <= 64 && (cin_group & 7) == 0 &&
           (pixel_stride & 7) == 0 && (channel_offset & 7) == 0;
}

int launch_igemm_thin(const GemmProblem &p, hipStream_t stream) {
    EH_REQUIRE(p.k_pad == 32 || p.k_pad == 64, "igemm_thin: padded reduction length %d", p.k_pad);
    EH_REQUIRE((p.k & 7) == 0 && (p.cin & 7) == 0 && (reinterpret_cast<uintptr_t>(p.a) & 7) == 0,
               "igemm_thin: rows must start on 8-byte boundaries");
    if (p.k_pad == 32) return launch_steps<1>(p, stream);
    return launch_steps<2>(p, stream);
}

}  // namespace eh
