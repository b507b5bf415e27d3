// One-tap problems (fully connected layers, 1x1 convolutions) on at most 64 rows of activations and a reduction longer
// than the one-tap kernel's: batch-1 ... batch-64 classifier heads.  Such a launch is the weights' one trip from memory
// and nothing else, so the work is cut along the WEIGHTS: a workgroup of eight waves owns 32 output channels, its waves
// take the 32-byte reduction steps round-robin, and a step's weight fragment is one contiguous KiB of the packed weights
// (MFMA fragment order, as for the one-tap kernel), fetched by one 16-byte-per-lane load straight into the registers the
// matrix instruction reads, eight such loads in flight per wave.  The activations (at most 64 rows, shared by every
// workgroup through the caches) are read in fragment form as well; rows past the last one multiply as zero.  The eight
// partial tiles and the rows' partial byte sums add up in LDS, and the first wave(s) requantize and store.
//
// Replaces, on these shapes, CLFullyConnected's float detour (gpu/operators/CLFullyConnected.cpp:22-150) and the
// reference's quantizedGemmBlocked (cl_kernels/ConvolutionKernels.cpp:956-1315), like the tiled kernels do on larger ones.
#include <type_traits>

#include "eh_internal.h"

namespace eh {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));

constexpr int kWaves = 8;    // waves of a workgroup, each on every eighth reduction step
constexpr int kFlight = 8;   // weight fragments a wave has on their way

// G: groups of 32 activation rows (1 or 2).  FAST: every requantization pair in use is inside the single-shift form's range.
template <int G, bool ROWSUM, bool FAST>
__global__ __launch_bounds__(kWaves * 64) void skinny_gemm_kernel(const GemmProblem p, const int ksteps) {
    __shared__ int32_t part_s[G][17][64];  // [group][accumulator, then the byte sum][lane]: where the waves' partial tiles add up
    const int tid = threadIdx.x, lane = tid & 63, r = lane & 31, half = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nb = blockIdx.x;
    for (int i = tid; i < G * 17 * 64; i += kWaves * 64) (&part_s[0][0][0])[i] = 0;
    __syncthreads();
    const v4i *wsrc = reinterpret_cast<const v4i *>(p.b) + (size_t)nb * ksteps * 64 + lane;
    // this lane's rows of the activation matrix, from its first reduction byte on
    const uint8_t *arow[G];
    bool row_ok[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const int row = g * 32 + r;
        row_ok[g] = row < p.m;
        arow[g] = p.a + (size_t)(row_ok[g] ? row : 0) * (size_t)p.cin + (size_t)p.a_offset + half * 16;
    }
    v16i acc[G];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[g][i] = 0;
    int rowsum[G];
#pragma unroll
    for (int g = 0; g < G; ++g) rowsum[g] = 0;

    for (int ks0 = wave; ks0 < ksteps; ks0 += kWaves * kFlight) {
        v4i bf[kFlight], af[kFlight][G];
#pragma unroll
        for (int u = 0; u < kFlight; ++u) {
            const int ks = ks0 + u * kWaves;
            const int ksc = ks < ksteps ? ks : ksteps - 1;  // (a step past the end: loaded again, not multiplied)
            bf[u] = wsrc[(size_t)ksc * 64];
            const int kb = ksc * 32 + half * 16;
#pragma unroll
            for (int g = 0; g < G; ++g) {
                // bytes past K (a reduction that ends inside its last step) and rows past M read as the byte that the flip turns into 0
                u32x4_a4 v = u32x4_a4{p.a_xor, p.a_xor, p.a_xor, p.a_xor};
                if (row_ok[g] && kb < p.k) v = *reinterpret_cast<const u32x4_a4 *>(arow[g] + ksc * 32);
                af[u][g] = v4i{(int)(v.x ^ p.a_xor), (int)(v.y ^ p.a_xor), (int)(v.z ^ p.a_xor), (int)(v.w ^ p.a_xor)};
            }
        }
#pragma unroll
        for (int u = 0; u < kFlight; ++u) {
            if (ks0 + u * kWaves < ksteps) {  // (uniform across the wave)
#pragma unroll
                for (int g = 0; g < G; ++g) {
                    if constexpr (ROWSUM) {
                        rowsum[g] = __builtin_amdgcn_sdot4(af[u][g].x, 0x01010101, rowsum[g], false);
                        rowsum[g] = __builtin_amdgcn_sdot4(af[u][g].y, 0x01010101, rowsum[g], false);
                        rowsum[g] = __builtin_amdgcn_sdot4(af[u][g].z, 0x01010101, rowsum[g], false);
                        rowsum[g] = __builtin_amdgcn_sdot4(af[u][g].w, 0x01010101, rowsum[g], false);
                    }
                    acc[g] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[u], af[u][g], acc[g], 0, 0, 0);
                }
            }
        }
    }
    // the partial tiles meet in LDS (integer adds: the order does not matter)
    if (wave < ksteps) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
#pragma unroll
            for (int i = 0; i < 16; ++i) atomicAdd(&part_s[g][i][lane], acc[g][i]);
            if constexpr (ROWSUM) atomicAdd(&part_s[g][16][lane], rowsum[g]);
        }
    }
    __syncthreads();
    if (wave >= G) return;
    const int g = wave;  // wave 0 finishes rows 0 .. 31, wave 1 rows 32 .. 63
    const int n = nb * 32 + half * 16;  // this lane's sixteen consecutive channels
    // the sixteen residual bytes these outputs are added to, requested before the requantization that hides their way
    u32x4_a4 res4 = u32x4_a4{0, 0, 0, 0};
    const bool res_vec = p.residual != nullptr && g * 32 + r < p.m && n + 16 <= p.n && (p.ldc & 3) == 0 &&
                         (reinterpret_cast<uintptr_t>(p.residual) & 3) == 0;
    if (res_vec) res4 = *reinterpret_cast<const u32x4_a4 *>(p.residual + (size_t)(g * 32 + r) * (size_t)p.ldc + n);
    int ncorr = 0;
    if constexpr (ROWSUM) {
        int rs = part_s[g][16][lane];
        rs += __shfl_xor(rs, 32);  // the other half of every step's bytes
        ncorr = -p.zw * rs;
    }
    int32_t x[16];
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
        const int4 bb = *reinterpret_cast<const int4 *>(p.bias + n + q4 * 4);  // (padded to whole channel blocks)
        x[q4 * 4 + 0] = bb.x;
        x[q4 * 4 + 1] = bb.y;
        x[q4 * 4 + 2] = bb.z;
        x[q4 * 4 + 3] = bb.w;
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) x[i] += ncorr + part_s[g][i][lane];
    const RequantDev rq = p.rq;
    uint32_t packed[4];
    auto produce = [&](auto mode_c) {
        constexpr int mode = decltype(mode_c)::value;
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
            if (rq.pc_multiplier) {  // (the arrays are padded past the last channel block)
                const int4 cm = *reinterpret_cast<const int4 *>(rq.pc_multiplier + n + q4 * 4);
                const int4 cs = *reinterpret_cast<const int4 *>(rq.pc_shift + n + q4 * 4);
                auto one = [&](int v, int32_t mult, int32_t shift) {
                    if constexpr (mode == 0)
                        return requant_u8_channel(v, mult, shift, rq);
                    else
                        return requant_u8_channel_fast<mode>(v, mult, shift, rq);
                };
                packed[q4] = pack_bytes(one(x[q4 * 4 + 0], cm.x, cs.x), one(x[q4 * 4 + 1], cm.y, cs.y), one(x[q4 * 4 + 2], cm.z, cs.z),
                                        one(x[q4 * 4 + 3], cm.w, cs.w)) ^
                             p.out_xor;
                continue;
            }
            if constexpr (mode != 0)
                packed[q4] = requant4_fast<mode>(x[q4 * 4 + 0], x[q4 * 4 + 1], x[q4 * 4 + 2], x[q4 * 4 + 3], 0, rq) ^ p.out_xor;
            else
                packed[q4] = pack_bytes(requant_u8_as<mode>(x[q4 * 4 + 0], rq), requant_u8_as<mode>(x[q4 * 4 + 1], rq),
                                        requant_u8_as<mode>(x[q4 * 4 + 2], rq), requant_u8_as<mode>(x[q4 * 4 + 3], rq)) ^
                             p.out_xor;
        }
    };
    if constexpr (!FAST)
        produce(std::integral_constant<int, 0>{});
    else if (rq.fast == 2)
        produce(std::integral_constant<int, 2>{});
    else
        produce(std::integral_constant<int, 1>{});
    const int row = g * 32 + r;
    if (row < p.m && n < p.n) {
        uint8_t *dst = p.out + (size_t)row * (size_t)p.ldc + n;
        const int cnt = p.n - n;
        if (p.residual) {  // out = add(residual, result)
            if (res_vec) {
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) packed[q4] = add_word(res4[q4], packed[q4], p.radd);
            } else {
                const uint8_t *res = p.residual + (size_t)row * (size_t)p.ldc + n;
                for (int t = 0; t < (cnt < 16 ? cnt : 16); ++t) {
                    const uint32_t v = add_one(res[t], (packed[t >> 2] >> (8 * (t & 3))) & 255u, p.radd);
                    packed[t >> 2] = (packed[t >> 2] & ~(255u << (8 * (t & 3)))) | (v << (8 * (t & 3)));
                }
            }
        }
        if (cnt >= 16 && (p.ldc & 3) == 0 && (reinterpret_cast<uintptr_t>(p.out) & 3) == 0) {
            *reinterpret_cast<u32x4_a4 *>(dst) = u32x4_a4{packed[0], packed[1], packed[2], packed[3]};
        } else {
            store_bytes_any_alignment(dst, packed, cnt < 16 ? cnt : 16);
        }
    }
}

}  // namespace

// One tap at the pixel itself over rows of whole 16-byte chunks, at most 64 output pixels, which the problem addresses as a
// plain matrix (pixel m reads at m * pixel_stride + channel_offset and writes at m * ldc), and a reduction beyond the
// one-tap kernel's.  Every workgroup reads all of the activations: beyond 32 rows that pays only while the channels are
// too few for the tiled kernels to spread (measured at 64 rows: 1280 -> 1000 channels 6.5 against 7.5 us, 4096 -> 4096
// 11.4 against 7.7 us).
bool gemm_skinny_applies(int32_t taps, int32_t cin_group, int32_t pixel_stride, int32_t channel_offset, int64_t m, int64_t n) {
    if (!(taps == 1 && m >= 1 && m <= 64 && cin_group > 256 && (cin_group & 15) == 0 && (pixel_stride & 15) == 0 && (channel_offset & 15) == 0)) return false;
    return m <= 32 || n <= 2048;
}

int launch_gemm_skinny(const GemmProblem &p, hipStream_t stream) {
    EH_REQUIRE(p.m >= 1 && p.m <= 64 && p.k_pad % 32 == 0 && p.k_pad >= p.k && (p.k & 15) == 0 && (p.cin & 15) == 0 && (p.a_offset & 15) == 0,
               "gemm_skinny: %d rows, reduction %d (padded %d), row stride %d", p.m, p.k, p.k_pad, p.cin);
    EH_REQUIRE((reinterpret_cast<uintptr_t>(p.a) & 15) == 0, "gemm_skinny: the activations must start on a 16-byte boundary");
    // pixel m of the problem is row m of a matrix: stride 1, no offsets, dense output
    EH_REQUIRE(p.stride_h == 1 && p.stride_w == 1 && p.y_base == 0 && p.x_base == 0 && p.h == p.ho && p.w == p.wo && p.out_sy == 1 && p.out_sx == 1 &&
                   p.out_y0 == 0 && p.out_x0 == 0 && p.out_h == p.ho && p.out_w == p.wo,
               "gemm_skinny: the problem is not a plain matrix product");
    const int n_blocks = (p.n + 31) / 32, ksteps = p.k_pad / 32;
    const bool rowsum = p.zw != 0, fast = p.rq.fast != 0;
    auto launch = [&](auto g_c) {
        constexpr int G = decltype(g_c)::value;
        const dim3 grid((unsigned)n_blocks), block(kWaves * 64);
        if (rowsum && fast)
            hipLaunchKernelGGL((skinny_gemm_kernel<G, true, true>), grid, block, 0, stream, p, ksteps);
        else if (rowsum)
            hipLaunchKernelGGL((skinny_gemm_kernel<G, true, false>), grid, block, 0, stream, p, ksteps);
        else if (fast)
            hipLaunchKernelGGL((skinny_gemm_kernel<G, false, true>), grid, block, 0, stream, p, ksteps);
        else
            hipLaunchKernelGGL((skinny_gemm_kernel<G, false, false>), grid, block, 0, stream, p, ksteps);
    };
    if (p.m <= 32)
        launch(std::integral_constant<int, 1>{});
    else
        launch(std::integral_constant<int, 2>{});
    EH_HIP(hipGetLastError());
    return EH_OK;
}

}  // namespace eh
