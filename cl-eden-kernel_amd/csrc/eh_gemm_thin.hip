// uint8 GEMM kernel for one-tap problems (1x1 convolutions, fully-connected layers)
// that are short of work for the tiled kernels: at most 64 reduction bytes
// (pointwise expansions such as 24 -> 144), or a small pixel count (the late
// layers of an image network, classifier heads).
//
// Such layers are bound by memory or by latency, not by the matrix cores, so
// nothing is staged in LDS and no workgroup-wide step exists: a wave owns 32
// output pixels and a group of 32-channel blocks, every lane fetches 16 reduction
// bytes of its pixel per 32-byte step straight into the 32x32x32 MFMA fragment
// layout (the bytes of a wave are one contiguous span when the pixels are), and
// the weights, packed in fragment order, are read per block and step as one
// coalesced 1 KiB wave load that stays in L2.  Four steps' worth of loads are
// requested before the first MFMA of the group.
// The weight fragment is the row operand and its rows are permuted within a
// 32-channel block (see packed_b_offset), so a lane ends up with 16 consecutive
// output channels of its pixel: requantize, pack, one 16-byte store.
#include <type_traits>

#include "eh_internal.h"

namespace eh {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

namespace {

template <int NBU, int KU, bool ROWSUM, bool FAST>
__global__ __launch_bounds__(256) void direct_gemm_kernel(const GemmProblem p, const int n_blocks, const int ksteps,
                                                          const int stage_out) {
    // KU: reduction steps whose loads are in flight together; NBU: channel blocks per wave
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
                 (size_t)p.a_offset;
        out_off = (((size_t)img * p.out_h + (oy * p.out_sy + p.out_y0)) * p.out_w + (ox * p.out_sx + p.out_x0)) * (size_t)p.ldc;
    }
    const uint8_t *arow = p.a + in_off + half * 16;
    const RequantDev rq = p.rq;
    const bool aligned16 = (p.ldc & 15) == 0 && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
    const v4i *bfrag = reinterpret_cast<const v4i *>(p.b) + lane;
    // stage_out: the 32 pixels of a wave are 32 * N contiguous output bytes (plain channels-last rows, N a
    // multiple of 8, one workgroup row per pixel block): the wave collects its rows in LDS and writes them
    // as one linear run of 16-byte pieces, whole cache lines instead of a 32-byte piece per pixel and block
    extern __shared__ __align__(16) uint8_t out_stage[];
    uint8_t *wave_stage = out_stage + (size_t)wave * 32 * p.n;

    // blockIdx.y spreads the channel-block groups over workgroups when there are few pixels
    for (int nb0 = blockIdx.y * NBU; nb0 < n_blocks; nb0 += gridDim.y * NBU) {
        const v4i *bblk[NBU];
        int4 bb[NBU][4];
#pragma unroll
        for (int u = 0; u < NBU; ++u) {
            const int nb = nb0 + u < n_blocks ? nb0 + u : n_blocks - 1;
            bblk[u] = bfrag + (size_t)nb * ksteps * 64;
#pragma unroll
            for (int g = 0; g < 4; ++g) bb[u][g] = *reinterpret_cast<const int4 *>(p.bias + nb * 32 + half * 16 + g * 4);
        }
        // SINGLE: the whole reduction is one group of KU steps, so each channel block's accumulator
        // can be formed right before it is requantized instead of all NBU living side by side
        constexpr bool SINGLE = KU < 4;
        v16i acc[SINGLE ? 1 : NBU];
        v4i afs[SINGLE ? KU : 1], bfs[SINGLE ? KU : 1][SINGLE ? NBU : 1];
        int rowsum = 0;
        for (int ks0 = 0; ks0 < (SINGLE ? 1 : ksteps); ks0 += KU) {
            // reduction bytes past K read as the byte that the sign flip turns into 0; steps past the
            // last one therefore multiply by zero whatever weight block they re-read
            uint2 lo[KU], hi[KU];
            v4i bf[KU][NBU];
#pragma unroll
            for (int t = 0; t < KU; ++t) {
                const int kb = (ks0 + t) * 32 + half * 16;
                lo[t] = make_uint2(p.a_xor, p.a_xor);
                hi[t] = lo[t];
                if (row_ok && kb < p.k) lo[t] = *reinterpret_cast<const uint2 *>(arow + (ks0 + t) * 32);
                if (row_ok && kb + 8 < p.k) hi[t] = *reinterpret_cast<const uint2 *>(arow + (ks0 + t) * 32 + 8);
                const int ks = ks0 + t < ksteps ? ks0 + t : ksteps - 1;
#pragma unroll
                for (int u = 0; u < NBU; ++u) bf[t][u] = bblk[u][ks * 64];
            }
            if constexpr (!SINGLE) {
                if (ks0 == 0) {
#pragma unroll
                    for (int u = 0; u < NBU; ++u)
#pragma unroll
                        for (int i = 0; i < 16; ++i) acc[u][i] = 0;
                }
            }
#pragma unroll
            for (int t = 0; t < KU; ++t) {
                v4i af;
                af.x = (int)(lo[t].x ^ p.a_xor);
                af.y = (int)(lo[t].y ^ p.a_xor);
                af.z = (int)(hi[t].x ^ p.a_xor);
                af.w = (int)(hi[t].y ^ p.a_xor);
                if constexpr (ROWSUM) {
                    rowsum = __builtin_amdgcn_sdot4(af.x, 0x01010101, rowsum, false);
                    rowsum = __builtin_amdgcn_sdot4(af.y, 0x01010101, rowsum, false);
                    rowsum = __builtin_amdgcn_sdot4(af.z, 0x01010101, rowsum, false);
                    rowsum = __builtin_amdgcn_sdot4(af.w, 0x01010101, rowsum, false);
                }
                if constexpr (SINGLE) {
                    afs[t] = af;
#pragma unroll
                    for (int u = 0; u < NBU; ++u) bfs[t][u] = bf[t][u];
                } else {
#pragma unroll
                    for (int u = 0; u < NBU; ++u) acc[u] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[t][u], af, acc[u], 0, 0, 0);
                }
            }
        }
        int ncorr = 0;
        if constexpr (ROWSUM) {
            rowsum += __shfl_xor(rowsum, 32);  // the other half of this pixel's reduction bytes
            ncorr = -p.zw * rowsum;
        }
#pragma unroll
        for (int u = 0; u < NBU; ++u) {
            const int nb = nb0 + u;
            if (nb >= n_blocks) break;
            const int n = nb * 32 + half * 16;  // this lane's 16 consecutive channels
            const int ai = SINGLE ? 0 : u;
            if constexpr (SINGLE) {
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[0][i] = 0;
#pragma unroll
                for (int t = 0; t < KU; ++t) acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bfs[t][u], afs[t], acc[0], 0, 0, 0);
            }
            uint32_t packed[4];
            auto quantize = [&](auto mode_c) {
                constexpr int mode = decltype(mode_c)::value;
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    uint32_t o0, o1, o2, o3;
                    if (mode == 0 && rq.pc_multiplier) {  // per-channel parameters (the padded arrays cover whole blocks)
                        const int32_t *pm = rq.pc_multiplier + n + g * 4;
                            const int4 cm = make_int4(pm[0], pm[1], pm[2], pm[3]);
                        const int32_t *ps = rq.pc_shift + n + g * 4;
                            const int4 cs = make_int4(ps[0], ps[1], ps[2], ps[3]);
                        o0 = requant_u8_channel(acc[ai][g * 4 + 0] + bb[u][g].x + ncorr, cm.x, cs.x, rq);
                        o1 = requant_u8_channel(acc[ai][g * 4 + 1] + bb[u][g].y + ncorr, cm.y, cs.y, rq);
                        o2 = requant_u8_channel(acc[ai][g * 4 + 2] + bb[u][g].z + ncorr, cm.z, cs.z, rq);
                        o3 = requant_u8_channel(acc[ai][g * 4 + 3] + bb[u][g].w + ncorr, cm.w, cs.w, rq);
                    } else {
                        o0 = requant_u8_as<mode>(acc[ai][g * 4 + 0] + bb[u][g].x + ncorr, rq);
                        o1 = requant_u8_as<mode>(acc[ai][g * 4 + 1] + bb[u][g].y + ncorr, rq);
                        o2 = requant_u8_as<mode>(acc[ai][g * 4 + 2] + bb[u][g].z + ncorr, rq);
                        o3 = requant_u8_as<mode>(acc[ai][g * 4 + 3] + bb[u][g].w + ncorr, rq);
                    }
                    packed[g] = (o0 | (o1 << 8) | (o2 << 16) | (o3 << 24)) ^ p.out_xor;
                }
            };
            if constexpr (!FAST)
                quantize(std::integral_constant<int, 0>{});
            else if (rq.fast == 2)
                quantize(std::integral_constant<int, 2>{});
            else
                quantize(std::integral_constant<int, 1>{});
            if (stage_out) {
                if (n < p.n) {
                    uint2 *dst2 = reinterpret_cast<uint2 *>(wave_stage + r * p.n + n);
                    dst2[0] = make_uint2(packed[0], packed[1]);
                    if (n + 8 < p.n) dst2[1] = make_uint2(packed[2], packed[3]);
                }
                continue;
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
    if (stage_out) {
        __syncthreads();
        const int m_wave = (blockIdx.x * 4 + wave) * 32;
        const int rows = p.m - m_wave < 32 ? p.m - m_wave : 32;
        const int bytes = rows > 0 ? rows * p.n : 0;  // a multiple of 8
        uint8_t *dst = p.out + (size_t)m_wave * p.n;   // 16-byte aligned: m_wave is a multiple of 32
        for (int off = lane * 16; off < bytes; off += 64 * 16) {
            if (off + 16 <= bytes) {
                *reinterpret_cast<uint4 *>(dst + off) = *reinterpret_cast<const uint4 *>(wave_stage + off);
            } else {
                *reinterpret_cast<uint2 *>(dst + off) = *reinterpret_cast<const uint2 *>(wave_stage + off);
            }
        }
    }
}

template <int NBU, int KU>
int launch_nbu(const GemmProblem &p, hipStream_t stream) {
    const int n_blocks = (p.n + 31) / 32, ksteps = p.k_pad / 32;
    // enough waves to fill 256 CUs several times over: with few pixels the channel-block groups are spread over grid.y too
    const int row_groups = (p.m + 127) / 128, n_groups = (n_blocks + NBU - 1) / NBU;
    int split = 1;
    while (split < n_groups && (long)row_groups * split < 2048) ++split;
    const dim3 grid(row_groups, split);
    // rows of one pixel block contiguous in the output (see the kernel): identity pixel mapping, no channel offset
    const bool linear = split == 1 && p.ldc == p.n && (p.n & 7) == 0 && p.n <= 384 && p.out_sy == 1 && p.out_sx == 1 &&
                        p.out_y0 == 0 && p.out_x0 == 0 && p.out_h == p.ho && p.out_w == p.wo &&
                        (reinterpret_cast<uintptr_t>(p.out) & 15) == 0;
    const int stage_out = linear ? 1 : 0;
    const size_t lds = linear ? (size_t)4 * 32 * p.n : 0;
    if (p.zw != 0) {
        if (p.rq.fast)
            hipLaunchKernelGGL((direct_gemm_kernel<NBU, KU, true, true>), grid, dim3(256), lds, stream, p, n_blocks, ksteps, stage_out);
        else
            hipLaunchKernelGGL((direct_gemm_kernel<NBU, KU, true, false>), grid, dim3(256), lds, stream, p, n_blocks, ksteps, stage_out);
    } else {
        if (p.rq.fast)
            hipLaunchKernelGGL((direct_gemm_kernel<NBU, KU, false, true>), grid, dim3(256), lds, stream, p, n_blocks, ksteps, stage_out);
        else
            hipLaunchKernelGGL((direct_gemm_kernel<NBU, KU, false, false>), grid, dim3(256), lds, stream, p, n_blocks, ksteps, stage_out);
    }
    EH_HIP(hipGetLastError());
    return EH_OK;
}

}  // namespace

// A single tap at the pixel itself (1x1 kernel, no padding) whose rows start on 8-byte
// boundaries, and either at most 64 reduction bytes, or at most 256 and so few multiply-adds
// overall that latency, not throughput, decides (the weights are re-read from L2 for every 32
// pixels, and a wave walks the whole reduction alone).
bool igemm_thin_applies(int32_t taps, int32_t cin_group, int32_t pixel_stride, int32_t channel_offset, int32_t y_base,
                        int32_t x_base, int64_t m, int64_t n) {
    if (!(taps == 1 && y_base == 0 && x_base == 0 && cin_group > 0 && (cin_group & 7) == 0 && (pixel_stride & 7) == 0 &&
          (channel_offset & 7) == 0))
        return false;
    return cin_group <= 64 || (cin_group <= 256 && m * n * cin_group <= 1500000000ll);
}

int launch_igemm_thin(const GemmProblem &p, hipStream_t stream) {
    EH_REQUIRE(p.k_pad % 32 == 0 && p.k_pad >= p.k, "igemm_thin: padded reduction length %d", p.k_pad);
    EH_REQUIRE((p.k & 7) == 0 && (p.cin & 7) == 0 && (reinterpret_cast<uintptr_t>(p.a) & 7) == 0,
               "igemm_thin: rows must start on 8-byte boundaries");
    const int n_blocks = (p.n + 31) / 32;
    if (p.k_pad == 32) {
        if (n_blocks == 1) return launch_nbu<1, 1>(p, stream);
        if (n_blocks == 2) return launch_nbu<2, 1>(p, stream);
        return launch_nbu<4, 1>(p, stream);
    }
    if (p.k_pad == 64) {
        if (n_blocks == 1) return launch_nbu<1, 2>(p, stream);
        if (n_blocks == 2) return launch_nbu<2, 2>(p, stream);
        return launch_nbu<4, 2>(p, stream);
    }
    if (n_blocks == 1) return launch_nbu<1, 4>(p, stream);
    return launch_nbu<2, 4>(p, stream);
}

}  // namespace eh
