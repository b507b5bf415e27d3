// Convolutions on one to four input channels with kernels of 3 to 11 rows (the first layer of an image network on RGB,
// RGBA or grey images: 7x7 stride 2, 5x5, 9x9 ...), channels-last uint8, any stride and padding, dilation 1, on the
// gfx950 matrix cores without an im2col buffer.
//
// The taps of one kernel row under an output pixel are kw * cin <= 32 CONTIGUOUS input bytes, so the reduction is laid
// out row by row: kernel row ky is reduction bytes [32 ky, 32 ky + kw cin), the rest of its 32 bytes zero (the weights
// are packed the same way, pack_weights_kernel with row_bytes).  One v_mfma_i32_32x32x32_i8 step is then one kernel row,
// and lane (r, half) of the step's activation fragment wants bytes [16 half, 16 half + 16) of pixel r's row: ONE
// unaligned 16-byte load straight from the image, no exchange between lanes and no staging.  Taps outside the image are
// replaced by the input zero point with a byte mask made from the pixel's first and last valid column (the same for all
// kernel rows), rows outside the image by the zero point as a whole; bytes past kw * cin are cleared.  Arithmetic is the
// implicit-GEMM one: a' = a ^ 0x80 against w - 128, zero-point terms folded into the bias, -(zp_w - 128) * sum a' per
// pixel from v_dot4 over the fragments, known before the first product, so the accumulators start from bias + that term.
//
// A workgroup stages the weight fragments of its range of output channels in LDS once ([block][row][lane], 1 KiB each)
// and its four waves walk 32-pixel blocks with stride (a persistent grid).  Stands in for the reference's direct 7x7 / 9x9 kernels
// (gpu/operators/CLConvolution.cpp:166-172, cl_kernels/DirectConvolutionKernel.cpp) and its GEMM path
// (CLGEMMConvolutionQuantized.cpp:33-280) on these shapes, where an im2col row would be mostly padding.
#include <atomic>
#include <type_traits>

#include "eh_internal.h"

namespace eh {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_a1 __attribute__((ext_vector_type(4), aligned(1)));
typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));

// bytes [lo, hi) of a dword as a mask (0 <= lo, hi <= 4 after clamping)
__device__ __forceinline__ uint32_t byte_range_mask(int lo, int hi) {
    lo = lo < 0 ? 0 : (lo > 4 ? 4 : lo);
    hi = hi < 0 ? 0 : (hi > 4 ? 4 : hi);
    if (hi <= lo) return 0u;
    const uint32_t upto_hi = hi == 4 ? 0xFFFFFFFFu : ((1u << (8 * hi)) - 1u);
    const uint32_t upto_lo = (1u << (8 * lo)) - 1u;  // lo < 4 here
    return upto_hi & ~upto_lo;
}

// KH: kernel rows.  FAST: every requantization pair in use is inside the single-shift form's range.
// The grid is persistent: as many workgroups as the device keeps resident (a multiple of 8); XCD x (workgroups x, x + 8,
// ...) walks the x-th contiguous eighth of the 32-pixel blocks, so the input rows that neighbouring output rows share are
// fetched into one L2 only, and a wave requests its next block's bytes before it multiplies the current one.
template <int KH, bool ROWSUM, bool FAST>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(KH <= 7 ? 4 : 3))) void conv_rows_kernel(const GemmProblem p, const uint32_t in_bytes, const int nbw, const int m_blocks) {
    extern __shared__ __align__(16) uint8_t lds_raw[];
    v4i *w_s = reinterpret_cast<v4i *>(lds_raw);  // [nbw][KH][64 lanes]
    int32_t *bias_s = reinterpret_cast<int32_t *>(lds_raw + (size_t)nbw * KH * 1024);  // [nbw * 32]
    const int tid = threadIdx.x, lane = tid & 63, r = lane & 31, half = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n_blocks = (p.n + 31) >> 5;
    const int nb_first = blockIdx.y * nbw;
    const int nb_count = n_blocks - nb_first < nbw ? n_blocks - nb_first : nbw;
    // weight rows are stored plainly, [channel][KH * 32 bytes]: row r of a fragment is channel 16 h + 4 g + t of its block
    for (int i = tid; i < nb_count * KH * 64; i += 256) {
        const int l = i & 63, s = (i >> 6) % KH, nb = (i >> 6) / KH;
        const int rr = l & 31;
        const int ch = (nb_first + nb) * 32 + 16 * ((rr >> 2) & 1) + 4 * (rr >> 3) + (rr & 3);
        w_s[i] = *reinterpret_cast<const v4i *>(p.b + (size_t)ch * (KH * 32) + s * 32 + (l >> 5) * 16);
    }
    for (int i = tid; i < nb_count * 32; i += 256) bias_s[i] = p.bias[nb_first * 32 + i];
    __syncthreads();
    const int xcd = (int)(blockIdx.x & 7u), per_xcd = (m_blocks + 7) >> 3;
    const int mb_end = (xcd + 1) * per_xcd < m_blocks ? (xcd + 1) * per_xcd : m_blocks;
    const int mb_stride = (int)(gridDim.x >> 3) * 4;
    const int plane = p.ho * p.wo;
    const int row_bytes = p.rows_kw * p.cin;
    const int row_pitch = p.w * p.cin;
    const RequantDev rq = p.rq;
    // bytes of this lane's sixteen that lie inside a kernel row at all; what an out-of-image tap contributes there
    uint32_t tail[4], fill_op[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        tail[d] = byte_range_mask(0 - (16 * half + 4 * d), row_bytes - (16 * half + 4 * d));
        fill_op[d] = (p.fill ^ p.a_xor) & tail[d];
    }

    // what a lane knows of its pixel of one 32-pixel block
    struct Pixel {
        bool m_ok;
        bool simple;         // (uniform across the wave) every window of the block lies wholly inside its image: no masks
        uint32_t rows_ok;    // bit s: kernel row s lies inside the image
        uint32_t inside[4];  // bytes of the lane's sixteen whose column lies inside the image (and inside the kernel row)
        size_t out_off;
    };
    const int image_bytes = p.h * row_pitch;
    const bool aligned_base = (reinterpret_cast<uintptr_t>(p.a) & 3) == 0;
    // Requests the raw bytes of block mb.  A row outside the image reads the nearest row inside instead (its bytes are
    // masked afterwards), so the loads need no branch; only a window that reaches before the first or past the last
    // byte of the whole tensor (first and last pixels of the first and last image) takes the nearest sixteen bytes
    // inside and shifts them.  (Rows, row pitch and pixel coordinates stay below 2^23, which the launcher checks: 24-bit
    // multiplies run at full rate, 32-bit ones at a quarter of it.)
    auto request = [&](int mb, Pixel &px, uint32_t (&raw)[KH][4]) {
        const int m_raw = mb * 32 + r;
        px.m_ok = m_raw < p.m;
        const int m = px.m_ok ? m_raw : p.m - 1;
        const int img = (int)fastdiv((uint32_t)m, p.div_plane), rem = m - img * plane;
        const int oy = (int)fastdiv((uint32_t)rem, p.div_wo), ox = rem - __mul24(oy, p.wo);
        const int iy0 = __mul24(oy, p.stride_h) + p.y_base, ix0 = __mul24(ox, p.stride_w) + p.x_base;
        const int pixel = (img * p.out_h + __mul24(oy, p.out_sy) + p.out_y0) * p.out_w + __mul24(ox, p.out_sx) + p.out_x0;
        px.out_off = (size_t)(uint32_t)pixel * (size_t)(uint32_t)p.ldc;
        const bool whole = iy0 >= 0 && iy0 + KH <= p.h && ix0 >= 0 && ix0 + p.rows_kw <= p.w;
        px.simple = __builtin_amdgcn_ballot_w64(!whole) == 0;
        const int a_img = img * image_bytes + __mul24(ix0, p.cin) + 16 * half;
        int a[KH];
        if (px.simple) {
#pragma unroll
            for (int s = 0; s < KH; ++s) a[s] = a_img + __mul24(iy0 + s, row_pitch);
        } else {
            // valid columns of the window: [c_lo, c_hi) -> valid bytes of a kernel row: [c_lo cin, c_hi cin)
            const int c_lo = ix0 < 0 ? -ix0 : 0;
            const int c_hi = p.w - ix0 < p.rows_kw ? p.w - ix0 : p.rows_kw;
            const int b_lo = c_lo * p.cin - 16 * half, b_hi = c_hi * p.cin - 16 * half;
#pragma unroll
            for (int d = 0; d < 4; ++d) px.inside[d] = byte_range_mask(b_lo - 4 * d, b_hi - 4 * d) & tail[d];
            px.rows_ok = 0;
#pragma unroll
            for (int s = 0; s < KH; ++s) {
                const int iy = iy0 + s;
                px.rows_ok |= (unsigned)iy < (unsigned)p.h ? 1u << s : 0u;
                const int iyc = iy < 0 ? 0 : (iy >= p.h ? p.h - 1 : iy);
                a[s] = a_img + __mul24(iyc, row_pitch);
            }
        }
        // (row addresses grow with s: the first and the last bound them all)
        // Sixteen bytes at any byte address as five aligned dwords funnelled together: lanes whose addresses are not
        // multiples of four cost the memory pipeline several times an aligned access (measured: 70 clocks per 16-byte
        // load of a wave against the extra dword and four v_alignbyte here).
        const bool in_tensor = a[0] >= 0 && ((uint32_t)a[KH - 1] & ~3u) + 20u <= in_bytes;
        if (__builtin_amdgcn_ballot_w64(!in_tensor) == 0 && aligned_base) {
#pragma unroll
            for (int s = 0; s < KH; ++s) {
                const uint8_t *src = p.a + (a[s] & ~3);
                const u32x4_a4 q = *reinterpret_cast<const u32x4_a4 *>(src);
                const uint32_t q4 = *reinterpret_cast<const uint32_t *>(src + 16);
                const uint32_t sh = (uint32_t)a[s] & 3u;
                raw[s][0] = __builtin_amdgcn_alignbyte(q.y, q.x, sh);
                raw[s][1] = __builtin_amdgcn_alignbyte(q.z, q.y, sh);
                raw[s][2] = __builtin_amdgcn_alignbyte(q.w, q.z, sh);
                raw[s][3] = __builtin_amdgcn_alignbyte(q4, q.w, sh);
            }
        } else {
            // sixteen bytes from the nearest address inside the tensor, moved to where they belong; what moves in is
            // zero and stands for bytes outside the tensor, which lie outside the image and are masked
#pragma unroll
            for (int s = 0; s < KH; ++s) {
                const int ac = a[s] < 0 ? 0 : ((uint32_t)a[s] + 16u > in_bytes ? (int)in_bytes - 16 : a[s]);
                const u32x4_a1 q = *reinterpret_cast<const u32x4_a1 *>(p.a + ac);
                const uint64_t lo = (uint64_t)q.x | ((uint64_t)q.y << 32), hi = (uint64_t)q.z | ((uint64_t)q.w << 32);
                const int bits = 8 * (a[s] - ac);  // > 0: the window starts behind ac (shift down), < 0: before it (shift up)
                uint64_t wlo = lo, whi = hi;
                if (bits >= 64) {
                    wlo = bits >= 128 ? 0 : hi >> (bits - 64);
                    whi = 0;
                } else if (bits > 0) {
                    wlo = (lo >> bits) | (hi << (64 - bits));
                    whi = hi >> bits;
                } else if (bits <= -64) {
                    whi = bits <= -128 ? 0 : lo << (-bits - 64);
                    wlo = 0;
                } else if (bits < 0) {
                    whi = (hi << -bits) | (lo >> (64 + bits));
                    wlo = lo << -bits;
                }
                raw[s][0] = (uint32_t)wlo;
                raw[s][1] = (uint32_t)(wlo >> 32);
                raw[s][2] = (uint32_t)whi;
                raw[s][3] = (uint32_t)(whi >> 32);
            }
        }
    };

    int mb = xcd * per_xcd + (int)(blockIdx.x >> 3) * 4 + wave;
    Pixel px;
    uint32_t raw[KH][4];
    if (mb < mb_end) request(mb, px, raw);
    for (; mb < mb_end; mb += mb_stride) {
        v4i af[KH];
        int rowsum = 0;
#pragma unroll
        for (int s = 0; s < KH; ++s) {
            uint32_t f[4];
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                if (px.simple) {
                    f[d] = (raw[s][d] ^ p.a_xor) & tail[d];
                } else {
                    const uint32_t keep = (px.rows_ok >> s) & 1u ? px.inside[d] : 0u;
                    f[d] = ((raw[s][d] ^ p.a_xor) & keep) | (fill_op[d] & ~keep);
                }
            }
            af[s] = v4i{(int)f[0], (int)f[1], (int)f[2], (int)f[3]};
            if constexpr (ROWSUM) {
#pragma unroll
                for (int d = 0; d < 4; ++d) rowsum = __builtin_amdgcn_sdot4((int)f[d], 0x01010101, rowsum, false);
            }
        }
        const bool m_ok = px.m_ok;
        const size_t out_off = px.out_off;
        if (mb + mb_stride < mb_end) request(mb + mb_stride, px, raw);  // (uniform across the wave)
        int ncorr = 0;
        if constexpr (ROWSUM) {
            rowsum += __shfl_xor(rowsum, 32);  // the other sixteen bytes of every kernel row
            ncorr = -p.zw * rowsum;
        }
        for (int nb = 0; nb < nb_count; ++nb) {
            const int n = (nb_first + nb) * 32 + half * 16;  // this lane's sixteen consecutive channels
            // the accumulators start from the folded bias and the pixel's row-sum term: nothing left to add afterwards
            v16i acc;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int4 bb = *reinterpret_cast<const int4 *>(bias_s + nb * 32 + half * 16 + g * 4);
                acc[g * 4 + 0] = bb.x + ncorr;
                acc[g * 4 + 1] = bb.y + ncorr;
                acc[g * 4 + 2] = bb.z + ncorr;
                acc[g * 4 + 3] = bb.w + ncorr;
            }
#pragma unroll
            for (int s = 0; s < KH; ++s) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(w_s[(nb * KH + s) * 64 + lane], af[s], acc, 0, 0, 0);
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
                        packed[g] = pack_bytes(one(acc[g * 4 + 0], cm.x, cs.x), one(acc[g * 4 + 1], cm.y, cs.y), one(acc[g * 4 + 2], cm.z, cs.z),
                                               one(acc[g * 4 + 3], cm.w, cs.w)) ^
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
            if (m_ok && n < p.n) {
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

constexpr int kRowsLdsMax = 48 * 1024;

}  // namespace

// One to four input channels (all of them: one group), kernel rows of at most 32 bytes, 3, 5, 7, 9 or 11 of them.
bool conv_rows_applies(int32_t cin_group, int32_t pixel_stride, int32_t kh, int32_t kw) {
    if (cin_group != pixel_stride || cin_group < 1 || cin_group > 4) return false;
    if (kw < 1 || kw * cin_group > 32) return false;
    return kh == 3 || kh == 5 || kh == 7 || kh == 9 || kh == 11;
}

int launch_conv_rows(const GemmProblem &p, hipStream_t stream) {
    EH_REQUIRE(conv_rows_applies(p.cin, p.cin, p.rows_kh, p.rows_kw) && p.k == p.rows_kh * p.rows_kw * p.cin && p.k_pad == p.rows_kh * 32,
               "conv_rows: not a few-channel problem of %d x %d taps on %d channels", p.rows_kh, p.rows_kw, p.cin);
    const size_t image_bytes = (size_t)p.h * p.w * p.cin;
    const int images = (p.m + p.ho * p.wo - 1) / (p.ho * p.wo);
    EH_REQUIRE(image_bytes * images < (1ull << 31) && image_bytes * images >= 16, "conv_rows: input of %zu bytes", image_bytes * images);
    EH_REQUIRE(p.h < (1 << 23) && (long)p.w * p.cin < (1l << 23) && p.ho < (1 << 23) && p.wo < (1 << 23) && (long)p.ho * p.stride_h < (1l << 23) &&
                   (long)p.wo * p.stride_w < (1l << 23) && (long)p.ho * p.out_sy < (1l << 23) && (long)p.wo * p.out_sx < (1l << 23) &&
                   (long)images * p.out_h * p.out_w < (1l << 31),
               "conv_rows: extents beyond the 24-bit products of the kernel's addressing");
    const uint32_t total_bytes = (uint32_t)(image_bytes * images);
    const int n_blocks = (p.n + 31) / 32;
    int nbw = kRowsLdsMax / (p.rows_kh * 1024 + 128);
    if (nbw > n_blocks) nbw = n_blocks;
    const int ranges = (n_blocks + nbw - 1) / nbw;
    const int m_blocks = (p.m + 31) / 32;
    const size_t lds = (size_t)nbw * p.rows_kh * 1024 + (size_t)nbw * 32 * sizeof(int32_t);
    const bool rowsum = p.zw != 0, fast = p.rq.fast != 0;
    // a persistent grid: what the device keeps resident of this variant (asked once per variant and KiB of LDS), at most
    // one workgroup per four pixel blocks, a multiple of 8
    auto grid_for = [&](auto kernel, std::atomic<int> *resident) {
        const size_t slot = (lds + 1023) / 1024;
        int per_cu = resident[slot].load(std::memory_order_relaxed);
        if (per_cu == 0) {
            int n = 0;
            if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, 256, lds) != hipSuccess || n < 1) n = 2;
            per_cu = n > 8 ? 8 : n;
            resident[slot].store(per_cu, std::memory_order_relaxed);
        }
        int wgs = (((m_blocks + 7) / 8 + 3) / 4) * 8;
        const int target = 256 * per_cu / ranges > 8 ? 256 * per_cu / ranges / 8 * 8 : 8;
        if (wgs > target) wgs = target;
        return dim3((unsigned)wgs, (unsigned)ranges);
    };
    auto launch = [&](auto kh_c) {
        constexpr int KH = decltype(kh_c)::value;
        static std::atomic<int> resident[4][50];
        if (rowsum && fast)
            hipLaunchKernelGGL((conv_rows_kernel<KH, true, true>), grid_for(conv_rows_kernel<KH, true, true>, resident[0]), dim3(256), lds, stream, p, total_bytes, nbw,
                               m_blocks);
        else if (rowsum)
            hipLaunchKernelGGL((conv_rows_kernel<KH, true, false>), grid_for(conv_rows_kernel<KH, true, false>, resident[1]), dim3(256), lds, stream, p, total_bytes, nbw,
                               m_blocks);
        else if (fast)
            hipLaunchKernelGGL((conv_rows_kernel<KH, false, true>), grid_for(conv_rows_kernel<KH, false, true>, resident[2]), dim3(256), lds, stream, p, total_bytes, nbw,
                               m_blocks);
        else
            hipLaunchKernelGGL((conv_rows_kernel<KH, false, false>), grid_for(conv_rows_kernel<KH, false, false>, resident[3]), dim3(256), lds, stream, p, total_bytes, nbw,
                               m_blocks);
    };
    switch (p.rows_kh) {
        case 3: launch(std::integral_constant<int, 3>{}); break;
        case 5: launch(std::integral_constant<int, 5>{}); break;
        case 7: launch(std::integral_constant<int, 7>{}); break;
        case 9: launch(std::integral_constant<int, 9>{}); break;
        default: launch(std::integral_constant<int, 11>{}); break;
    }
    EH_HIP(hipGetLastError());
    return EH_OK;
}

}  // namespace eh
