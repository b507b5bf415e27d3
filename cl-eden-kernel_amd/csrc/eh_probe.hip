// Measured ceilings of the machine the roofline figures are set against: the
// issue rate of the int8 MFMA this library uses, from registers only (no memory
// traffic at all).  With operand bits that toggle like real data the sustained
// clock under this load is lower than with constant operands, so both are
// reported.  And what plain streaming kernels reach on the byte ratios of the HBM-bound layers.
// Measurement utilities: they have no counterpart in the reference.
#include <utility>

#include "eh_internal.h"

namespace eh {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void mfma_i8_probe_kernel(const int iters, int *sink, const uint32_t scramble) {
    // scramble == 0: every operand register holds the same small constants
    const uint32_t h = (threadIdx.x + 1u) * 2654435761u * scramble;
    v4i a = {(int)(h + 1u), (int)(h * 31u + 7u), (int)((h * 17u) ^ 0x5bd1e995u), (int)(h * 101u + 3u)};
    v4i b = {(int)(h * 3u + 11u), (int)(h * h + 5u), (int)(h ^ 0x9e3779b9u), (int)(h * 7u + 2u)};
    v16i c0, c1, c2, c3;
#pragma unroll
    for (int i = 0; i < 16; ++i) c0[i] = c1[i] = c2[i] = c3[i] = 0;
    for (int i = 0; i < iters; ++i) {
        c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c3, 0, 0, 0);
    }
    sink[blockIdx.x * 256 + threadIdx.x] = c0[0] + c1[1] + c2[2] + c3[3];
}

// Streaming yardsticks for the HBM-bound kernels: 16 bytes per lane, whole lines per wave, nothing but the moves.
// MODE 0: copy.  MODE 1: every source chunk is written six times (the byte ratio of a 24 -> 144 pointwise layer).
// MODE 2: four source chunks are folded into one written chunk (the byte ratio of a stride-2 depthwise layer).
template <int MODE>
__global__ __launch_bounds__(256) void stream_probe_kernel(const uint4 *__restrict__ in, uint4 *__restrict__ out, const uint32_t n_out) {
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < n_out; i += gridDim.x * 256u) {
        if constexpr (MODE == 0) {
            out[i] = in[i];
        } else if constexpr (MODE == 1) {
            const uint4 a = in[i / 6u];
            out[i] = make_uint4(a.x + i, a.y, a.z, a.w);
        } else {
            const uint4 a = in[4u * i], b = in[4u * i + 1u], c = in[4u * i + 2u], d = in[4u * i + 3u];
            out[i] = make_uint4(a.x ^ b.x ^ c.x ^ d.x, a.y ^ b.y ^ c.y ^ d.y, a.z ^ b.z ^ c.z ^ d.z, a.w ^ b.w ^ c.w ^ d.w);
        }
    }
}

// What the matrix pipe of a CU can be fed with.  A workgroup of four waves (one per SIMD, as in the GEMM kernels) repeats
// an iteration of NM matrix instructions, NR 16-byte-per-lane LDS fragment reads, ND direct-to-LDS loads of 1 KiB
// (global_load_lds_dwordx4 from a region that stays in the XCD's L2) and NV ordinary 1 KiB loads into registers that
// SHARE waves request alike (an operand kept out of LDS), DEPTH iterations in flight, a barrier every SYNC iterations
// (0: none).  The proportions are those of the GEMM tiles' inner loops; the times say how far below the matrix
// instructions' own rate the feeding alone puts a tile shape, before any epilogue.
typedef __attribute__((address_space(3))) uint8_t lds_byte;

__device__ __forceinline__ void probe_dma16(const void *base_uniform, uint32_t lane_offset, uint32_t lds_base_uniform) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_offset), "s"(base_uniform), "s"(lds_base_uniform) : "memory");
}
__device__ __forceinline__ v4i probe_dsread(uint32_t a) {
    v4i r;
    asm volatile("ds_read_b128 %0, %1" : "=v"(r) : "v"(a) : "memory");
    return r;
}
template <int N>
__device__ __forceinline__ void probe_wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
template <int... I, class F>
__device__ __forceinline__ void probe_for_impl(std::integer_sequence<int, I...>, F &&f) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void probe_for(F &&f) {
    probe_for_impl(std::make_integer_sequence<int, N>{}, f);
}

constexpr uint32_t kFeedRegion = 1u << 20;  // bytes of source per XCD: stays in its 4 MiB L2

template <int NM, int NR, int ND, int NV, int SHARE, int SYNC>
__global__ __launch_bounds__(256) void feed_probe_kernel(const uint8_t *src, const int iters, int *sink) {
    constexpr int DEPTH = 4;
    constexpr uint32_t region_mask = kFeedRegion - 1;
    __shared__ __align__(1024) uint8_t lds[128 * 1024];  // fragment reads in the lower half, DMA destinations in the upper
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    for (int i = tid; i < 128 * 256; i += 256) reinterpret_cast<int *>(lds)[i] = (int)(i * 2654435761u);
    __syncthreads();
    const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_byte *)lds;
    const uint8_t *base = src + (size_t)(blockIdx.x & 7) * kFeedRegion;
    uint32_t goff = ((blockIdx.x >> 3) * 65536u + wave * 1024u + lane * 16u) & region_mask;
    uint32_t voff = ((blockIdx.x >> 3) * 65536u + 32768u + (wave / SHARE) * 1024u + lane * 16u) & region_mask;
    const int frow = lane & 31, fhalf = lane >> 5;
    const uint32_t raddr = lds0 + wave * 16384 + frow * 128 + ((fhalf ^ (frow & 7)) << 4);
    v16i acc[4];
    for (int q = 0; q < 4; ++q)
        for (int r = 0; r < 16; ++r) acc[q][r] = 0;
    const v4i fa = {tid, tid * 3, tid * 7, tid * 11};
    v4i fr[NR > 0 ? NR : 1];
    v4i vg[DEPTH][NV > 0 ? NV : 1];
    for (int d = 0; d < DEPTH; ++d)
        for (int j = 0; j < (NV > 0 ? NV : 1); ++j) vg[d][j] = fa;
    for (int j = 0; j < (NR > 0 ? NR : 1); ++j) fr[j] = fa;
    uint32_t ring = 0;
    for (int it = 0; it < iters; it += DEPTH) {
        probe_for<DEPTH>([&](auto d_c) {
            constexpr int d = decltype(d_c)::value;
            // this iteration's memory operations are consumed DEPTH - 1 iterations later
            probe_for<ND>([&](auto) {
                probe_dma16(base, goff, lds0 + 65536 + ((ring + wave * 1024) & 0xFFFF));
                ring += 4096;
                goff = (goff + 4096u) & region_mask;
            });
            constexpr int slot = (d + DEPTH - 1) % DEPTH;
            // (ordinary loads: the compiler tracks their registers and waits)
            probe_for<NV>([&](auto j_c) {
                vg[slot][decltype(j_c)::value] = *reinterpret_cast<const v4i *>(base + voff);
                voff = (voff + 4096u) & region_mask;
            });
            probe_for<NM>([&](auto q_c) {
                constexpr int q = decltype(q_c)::value;
                const v4i b = NV > 0 ? vg[d][q % (NV > 0 ? NV : 1)] : fa;
                const v4i a = NR > 0 ? fr[q % (NR > 0 ? NR : 1)] : fa;
                acc[q & 3] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc[q & 3], 0, 0, 0);
                if constexpr (NR > 0 && q < NR) fr[q] = probe_dsread(raddr);
            });
            if constexpr (NM == 0) probe_for<NR>([&](auto q_c) { fr[decltype(q_c)::value] = probe_dsread(raddr); });
            if constexpr (NR > 0) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if constexpr (ND + NV > 0) probe_wait_vmcnt<(DEPTH - 1) * (ND + NV)>();
            if constexpr (SYNC > 0) {
                if constexpr (d % SYNC == SYNC - 1) __syncthreads();
            }
        });
    }
    probe_wait_vmcnt<0>();
    int s = acc[0][0] + acc[1][1] + acc[2][2] + acc[3][3] + fa.x + lds[65536 + tid];
    for (int d = 0; d < DEPTH; ++d) s += vg[d][0].x;
    for (int j = 0; j < (NR > 0 ? NR : 1); ++j) s += fr[j].x;
    sink[blockIdx.x * 256 + tid] = s;
}

struct FeedMix {
    int mfma, lds_reads, dma, reg_loads;
    void (*kernel)(const uint8_t *, int, int *);
};
const FeedMix kFeedMixes[] = {
    {0, 0, 4, 0, feed_probe_kernel<0, 0, 4, 0, 1, 0>},    // 0: direct-to-LDS loads alone
    {0, 8, 0, 0, feed_probe_kernel<0, 8, 0, 0, 1, 0>},    // 1: fragment reads alone
    {4, 0, 0, 0, feed_probe_kernel<4, 0, 0, 0, 1, 0>},    // 2: matrix instructions alone
    {4, 4, 2, 0, feed_probe_kernel<4, 4, 2, 0, 1, 4>},    // 3: 128 x 128 tile, 128-byte slabs
    {4, 4, 4, 0, feed_probe_kernel<4, 4, 4, 0, 1, 2>},    // 4: 64 x 64 tile with the reduction split over the waves, 256-byte slabs
    {8, 6, 3, 0, feed_probe_kernel<8, 6, 3, 0, 1, 4>},    // 5: 256 x 128 tile
    {16, 8, 4, 0, feed_probe_kernel<16, 8, 4, 0, 1, 4>},  // 6: 256 x 256 tile
    {4, 2, 1, 2, feed_probe_kernel<4, 2, 1, 2, 2, 4>},    // 7: 128 x 128 with the weight operand straight into registers
    {16, 4, 2, 4, feed_probe_kernel<16, 4, 2, 4, 2, 4>},  // 8: 256 x 256 likewise
};

}  // namespace
}  // namespace eh

using namespace eh;

extern "C" int eh_probe_feed(int32_t mix, int32_t workgroups, int32_t iterations, double *ns_per_iteration, int32_t *per_iteration) {
    constexpr int MIXES = (int)(sizeof(kFeedMixes) / sizeof(kFeedMixes[0]));
    EH_REQUIRE(mix >= 0 && mix < MIXES && ns_per_iteration != nullptr, "feed probe: mix 0 .. %d", MIXES - 1);
    EH_REQUIRE(workgroups >= 1 && workgroups <= 4096 && iterations >= 4 && iterations <= (1 << 20) && iterations % 4 == 0,
               "feed probe: 1 .. 4096 workgroups, a multiple of four iterations up to 2^20");
    const FeedMix &m = kFeedMixes[mix];
    if (per_iteration) {
        per_iteration[0] = m.mfma;
        per_iteration[1] = m.lds_reads;
        per_iteration[2] = m.dma;
        per_iteration[3] = m.reg_loads;
    }
    uint8_t *src = nullptr;
    int *sink = nullptr;
    EH_HIP(hipMalloc(reinterpret_cast<void **>(&src), 8ull * kFeedRegion + 65536));
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&sink), (size_t)workgroups * 256 * sizeof(int));
    if (e != hipSuccess) {
        (void)hipFree(src);
        return hip_fail(e, "hipMalloc(feed probe sink)");
    }
    (void)hipMemset(src, 1, 8ull * kFeedRegion + 65536);
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    hipLaunchKernelGGL(m.kernel, dim3(workgroups), dim3(256), 0, 0, src, 64, sink);  // warm-up: the region is in L2 afterwards
    (void)hipEventRecord(e0, 0);
    hipLaunchKernelGGL(m.kernel, dim3(workgroups), dim3(256), 0, 0, src, iterations, sink);
    (void)hipEventRecord(e1, 0);
    e = hipEventSynchronize(e1);
    float ms = 0;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(sink);
    (void)hipFree(src);
    if (e != hipSuccess) return hip_fail(e, "feed probe");
    *ns_per_iteration = (double)ms * 1e6 / iterations;
    return EH_OK;
}

extern "C" int eh_probe_stream(const void *src, void *dst, int64_t out_bytes, int32_t mode, void *stream) {
    EH_REQUIRE(src && dst && out_bytes > 0 && (out_bytes & 15) == 0 && out_bytes < (1ll << 35), "stream probe: %lld bytes", (long long)out_bytes);
    EH_REQUIRE(mode >= 0 && mode <= 2, "stream probe: mode %d", mode);
    EH_REQUIRE(((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0, "stream probe: unaligned pointers");
    const uint32_t n_out = (uint32_t)(out_bytes / 16);
    const uint32_t blocks = (n_out + 255u) / 256u;
    const dim3 grid(blocks < 8192u ? blocks : 8192u);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint4 *in = static_cast<const uint4 *>(src);
    uint4 *out = static_cast<uint4 *>(dst);
    if (mode == 0)
        hipLaunchKernelGGL(stream_probe_kernel<0>, grid, dim3(256), 0, st, in, out, n_out);
    else if (mode == 1)
        hipLaunchKernelGGL(stream_probe_kernel<1>, grid, dim3(256), 0, st, in, out, n_out);
    else
        hipLaunchKernelGGL(stream_probe_kernel<2>, grid, dim3(256), 0, st, in, out, n_out);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

extern "C" int eh_probe_mfma_i8(int32_t iterations, int32_t toggling_operands, double *tops) {
    EH_REQUIRE(tops != nullptr && iterations > 0 && iterations <= (1 << 22), "probe: bad arguments");
    constexpr int WGS = 256;  // one workgroup of four waves per CU: one wave per SIMD
    int *sink = nullptr;
    EH_HIP(hipMalloc(reinterpret_cast<void **>(&sink), (size_t)WGS * 256 * sizeof(int)));
    hipEvent_t e0, e1;
    EH_HIP(hipEventCreate(&e0));
    EH_HIP(hipEventCreate(&e1));
    const uint32_t scramble = toggling_operands ? 1u : 0u;
    hipLaunchKernelGGL(mfma_i8_probe_kernel, dim3(WGS), dim3(256), 0, 0, 64, sink, scramble);  // warm-up
    EH_HIP(hipEventRecord(e0, 0));
    hipLaunchKernelGGL(mfma_i8_probe_kernel, dim3(WGS), dim3(256), 0, 0, iterations, sink, scramble);
    EH_HIP(hipEventRecord(e1, 0));
    EH_HIP(hipEventSynchronize(e1));
    float ms = 0;
    EH_HIP(hipEventElapsedTime(&ms, e0, e1));
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(sink);
    const double mfmas = (double)WGS * 4 * (double)iterations * 4;
    *tops = mfmas * (2.0 * 32 * 32 * 32) / ((double)ms * 1e-3) / 1e12;
    return EH_OK;
}
