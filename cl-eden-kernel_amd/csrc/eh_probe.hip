// Measured ceilings of the machine the roofline figures are set against: the
// issue rate of the int8 MFMA this library uses, from registers only (no memory
// traffic at all).  With operand bits that toggle like real data the sustained
// clock under this load is lower than with constant operands, so both are
// reported.  And what plain streaming kernels reach on the byte ratios of the HBM-bound layers.
// Measurement utilities: they have no counterpart in the reference.
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

}  // namespace
}  // namespace eh

using namespace eh;

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
