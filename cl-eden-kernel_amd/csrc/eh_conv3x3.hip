// 3x3 convolution, stride 1, dilation 1, uint8 channels-last, on the gfx950 matrix cores with the input patch
// staged in LDS once.
//
// The implicit-GEMM kernels fetch every input byte once per tap (nine times through a CU's L1).  Here a workgroup
// owns TH whole output rows of one image and a range of 32 or 64 output channels: it brings the (TH + 2) x (W_out + 2)
// input pixels those rows touch into LDS with wave-wide direct-to-LDS loads (pixels outside the image fetch the
// 16-byte constant that holds the input zero point, as the reference's pad pass writes it,
// gpu/operators/cl_optimized_impls/CLPadConvert.cpp:185), together with its channels' weights in MFMA fragment
// order, and the nine taps then read their 32x32x32 fragments from the same patch at shifted addresses.  Stands in
// for the reference's direct3x3 kernels, which likewise read an input pixel once per output-channel group and reuse
// it over the taps (gpu/operators/cl_kernels/DirectConvolutionKernel.cpp:4324-4869).
//
// LDS patch layout: pixel q = row * (W_out + 2) + column at byte q * pitch, pitch = C + 16 (C a multiple of 32) or
// C + 32 (C = 16 mod 32): the slack makes the pitch an odd number of 16-byte chunks, so the sixteen lanes that read one chunk
// position of sixteen consecutive pixels fall on sixteen distinct bank groups, and the fragment address of tap
// (ky, kx), channel offset c is the lane's base address plus one per-step constant.  The slack chunks are never
// fetched (their lanes are masked off) and never read.
//
// A wave takes up to four 32-pixel groups of the tile at a time: per 32-byte reduction step it reads the weight
// fragments of its one or two channel blocks once and one activation fragment per group, so a fragment read feeds
// two matrix instructions on average and the LDS port stays below the matrix cores' demand.  Arithmetic is the
// implicit-GEMM one (a' = a ^ 0x80 against w - 128, zero-point terms folded into the bias, -(zp_w - 128) * sum a'
// per pixel from v_dot4 over the same fragments); a lane ends up with 16 consecutive channels of one pixel.
#include <type_traits>

#include <atomic>

#include "eh_internal.h"

namespace eh {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) uint8_t lds_byte;

namespace {


__device__ __forceinline__ uint32_t lds_offset(const void *p) { return (uint32_t)(uintptr_t)(lds_byte *)p; }

// One wave copies up to 64 x 16 bytes: active lane i's 16 bytes land at lds_base + 16 * i.
__device__ __forceinline__ void dma16(const void *gptr, uint32_t lds_base_uniform) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gptr), "s"(lds_base_uniform) : "memory");
}

struct Conv3Launch {
    int32_t th;               // output rows per tile
    int32_t tiles_per_image;  // ceil(ho / th)
    int32_t tiles;            // n * tiles_per_image
    int32_t ksteps;           // ceil(9 * cin / 32)
    int32_t pitch;            // LDS bytes per patch pixel: cin + 16 or + 32 (conv3_pitch)
    int32_t pc;               // patch columns: wo + 2
    FastDiv div_pch, div_pc, div_wo, div_tiles;
};

// NB: 32-channel blocks per workgroup (grid y walks the channel ranges).
// QM: 0 two-step requantization (one pair, or one per channel), 1 / 2 the single-shift forms (2: no sign test).
// PC: one multiplier and shift per output channel.
// G: 32-pixel groups a wave multiplies together (4 where a tile has sixteen groups or more, fewer on small tiles, so
// that no matrix instruction is spent on repeated pixels).
// SPLIT (NB == 2 only): a wave works on ONE of the two channel blocks, the waves forming 2 x 2 over (pixel group,
// channel block): tiles of two pixel groups then keep all four waves busy instead of two.
template <int NB, bool ROWSUM, int QM, bool PC, int G = 4, bool SPLIT = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void conv3x3_patch_kernel(const GemmProblem p, const Conv3Launch L) {
    extern __shared__ __align__(1024) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, r = lane & 31, half = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // every XCD takes one contiguous eighth of the tiles: the rows two neighbouring tiles share are fetched into one L2
    const int tile = (int)((blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3));
    if (tile >= L.tiles) return;
    const int img = (int)fastdiv((uint32_t)tile, L.div_tiles);
    const int oy0 = (tile - img * L.tiles_per_image) * L.th;
    const int rows = p.ho - oy0 < L.th ? p.ho - oy0 : L.th;  // output rows of this tile
    const int pixels = rows * p.wo;
    const int nb_first = blockIdx.y * NB;
    const int n_blocks = (p.n + 31) >> 5;
    const int nb_count = n_blocks - nb_first < NB ? n_blocks - nb_first : NB;
    const int KS = L.ksteps;

    // LDS: weights [NB][KS][64 lanes][16 B] | bias [NB * 32] | step table [KS][2] | patch
    v4i *w_s = reinterpret_cast<v4i *>(lds);
    int32_t *bias_s = reinterpret_cast<int32_t *>(lds + (size_t)NB * KS * 1024);
    int32_t *step_s = bias_s + NB * 32;
    const uint32_t patch_off = (uint32_t)(((size_t)NB * KS * 1024 + NB * 128 + (size_t)KS * 8 + 1023) & ~(size_t)1023);
    uint8_t *patch = lds + patch_off;

    // ---- stage: weights (a linear copy of the packed fragment image), the patch, bias and step table
    {
        const uint8_t *wsrc = reinterpret_cast<const uint8_t *>(p.b) + (size_t)nb_first * KS * 1024;
        const int w_instr = nb_count * KS;  // 1 KiB each
        for (int i = wave; i < w_instr; i += 4) dma16(wsrc + (size_t)i * 1024 + lane * 16, lds_offset(lds) + (uint32_t)i * 1024u);
        const int pch = L.pitch >> 4, cpp = p.cin >> 4;  // chunks per pixel with and without the slack
        const int patch_pixels = (rows + 2) * L.pc;
        const int chunks = patch_pixels * pch;
        const int iy0 = oy0 + p.y_base, ix0 = p.x_base;
        const uint8_t *image = p.a + (size_t)img * p.h * p.w * p.cin;
        for (int i = wave; i * 64 < chunks; i += 4) {
            const int c = i * 64 + lane;
            const int q = (int)fastdiv((uint32_t)c, L.div_pch), ph = c - q * pch;
            if (q < patch_pixels && ph < cpp) {
                const int pr = (int)fastdiv((uint32_t)q, L.div_pc), pcx = q - pr * L.pc;
                const int iy = iy0 + pr, ix = ix0 + pcx;
                const bool inside = (unsigned)iy < (unsigned)p.h && (unsigned)ix < (unsigned)p.w;
                const uint8_t *src = inside ? image + ((size_t)(iy * p.w + ix) * p.cin + ph * 16) : p.fillbuf;
                dma16(src, lds_offset(patch) + (uint32_t)i * 1024u);
            }
        }
        if (tid < nb_count * 32) bias_s[tid] = p.bias[nb_first * 32 + tid];
        if (tid < KS * 2) {
            // reduction bytes [16 tid, 16 tid + 16) belong to tap koff / cin, channels koff % cin ...
            const int koff = tid * 16;
            const int tap = koff / p.cin, c0 = koff - tap * p.cin;
            const int ky = tap / 3, kx = tap - ky * 3;
            // (the half step past the ninth tap of a 16 (mod 32) channel count multiplies zero weights: any bytes will do)
            step_s[tid] = tap < 9 ? (ky * L.pc + kx) * L.pitch + c0 : 0;
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        // One pass over the patch in place: bytes to the signed operands the matrix cores take (a ^ 0x80), and each
        // pixel's sum of them over the channels into the pixel's slack chunk.  The nine taps then need neither a flip
        // nor a dot product per fragment: an output pixel's activation sum is nine of these pixel sums.
        if (ROWSUM || p.a_xor != 0) {
            const int a_flip = (int)p.a_xor;
            for (int q = tid; q < patch_pixels; q += 256) {
                uint8_t *px = patch + (size_t)q * L.pitch;
                v4i v[8];  // up to 128 channels; all of a pixel's chunks are read before the first is used
#pragma unroll
                for (int ch = 0; ch < 8; ++ch)
                    if (ch < cpp) v[ch] = *reinterpret_cast<v4i *>(px + ch * 16);
                int sum = 0;
#pragma unroll
                for (int ch = 0; ch < 8; ++ch) {
                    if (ch < cpp) {
                        v[ch].x ^= a_flip;
                        v[ch].y ^= a_flip;
                        v[ch].z ^= a_flip;
                        v[ch].w ^= a_flip;
                        if constexpr (ROWSUM) {
                            sum = __builtin_amdgcn_sdot4(v[ch].x, 0x01010101, sum, false);
                            sum = __builtin_amdgcn_sdot4(v[ch].y, 0x01010101, sum, false);
                            sum = __builtin_amdgcn_sdot4(v[ch].z, 0x01010101, sum, false);
                            sum = __builtin_amdgcn_sdot4(v[ch].w, 0x01010101, sum, false);
                        }
                        *reinterpret_cast<v4i *>(px + ch * 16) = v[ch];
                    }
                }
                if constexpr (ROWSUM) *reinterpret_cast<int *>(px + p.cin) = sum;
            }
            __syncthreads();
        }
    }

    const RequantDev rq = p.rq;
    const int groups = (pixels + 31) >> 5;
    const size_t out_tile = ((size_t)img * p.ho + oy0) * p.wo * (size_t)p.ldc;
    const bool wide = (p.ldc & 15) == 0 && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);

    // Wave w takes groups w', w' + 4, w' + 8, ... in passes of up to G.  When the groups do not divide by four the
    // first of them carry one more; w' is the wave number rotated by the workgroup's round of 256, so that the two
    // workgroups that share a CU put their longer waves on different SIMDs.
    static_assert(!SPLIT || NB == 2, "the split over channel blocks is written for two blocks");
    constexpr int NBW = SPLIT ? 1 : NB;        // channel blocks a wave works on
    constexpr int GW = SPLIT ? 2 : 4;          // waves side by side along the pixel groups
    const int wave_rot = (wave + (int)(blockIdx.x >> 8)) & 3;
    const int nb_lo = SPLIT ? wave_rot >> 1 : 0;
    for (int g0 = SPLIT ? (wave_rot & 1) : wave_rot; g0 < groups; g0 += GW * G) {
        int ng = (groups - g0 + GW - 1) / GW;  // groups of this pass that exist
        ng = ng < G ? ng : G;
        uint32_t base[G];   // patch byte address of the lane's pixel (top-left tap)
#pragma unroll
        for (int g = 0; g < G; ++g) {
            int pidx = (g0 + GW * g) * 32 + r;
            // (groups past the tile's last one repeat its last pixel and store nothing)
            pidx = pidx < pixels ? pidx : pixels - 1;
            const int py = (int)fastdiv((uint32_t)pidx, L.div_wo), px = pidx - py * p.wo;
            base[g] = (uint32_t)((py * L.pc + px) * L.pitch);
        }
        v16i acc[G][NBW];
#pragma unroll
        for (int nb = 0; nb < NBW; ++nb) {
            const int32_t *bsrc = bias_s + (nb_lo + nb) * 32 + half * 16;
            v16i b16;
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const int4 bb = *reinterpret_cast<const int4 *>(bsrc + q4 * 4);
                b16[q4 * 4 + 0] = bb.x;
                b16[q4 * 4 + 1] = bb.y;
                b16[q4 * 4 + 2] = bb.z;
                b16[q4 * 4 + 3] = bb.w;
            }
#pragma unroll
            for (int g = 0; g < G; ++g) acc[g][nb] = b16;
        }
        // -(zp_w - 128) * sum of the pixel's 9 * C signed activations.  The per-tensor single-shift forms take it inside
        // their rounding term, in the epilogue (one multiply-add per pixel and no register held across the products);
        // otherwise the accumulators start from it, so the epilogue has nothing left to add
        constexpr bool late_corr = ROWSUM && QM != 0 && !PC;
        auto pixel_term = [&](int g) {
            int rs = 0;
#pragma unroll
            for (int t = 0; t < 9; ++t) rs += *reinterpret_cast<const int *>(patch + base[g] + ((t / 3) * L.pc + t % 3) * L.pitch + p.cin);
            return -p.zw * rs;
        };
        if constexpr (ROWSUM && !late_corr) {
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const int ncorr = pixel_term(g);
#pragma unroll
                for (int nb = 0; nb < NBW; ++nb)
#pragma unroll
                    for (int i = 0; i < 16; ++i) acc[g][nb][i] += ncorr;
            }
        }

        // The fragments of step ks + 1 are requested before step ks is multiplied: the reads fly under the matrix
        // instructions, and the SIMD's other wave (two workgroups share a CU) fills what gaps remain.
        v4i af[2][G], bf[2][NBW];
        auto read_step = [&](int ks, auto buf_c) {
            constexpr int buf = decltype(buf_c)::value;
            const uint32_t d = (uint32_t)step_s[ks * 2 + half];
#pragma unroll
            for (int nb = 0; nb < NBW; ++nb) bf[buf][nb] = w_s[((nb_lo + nb < nb_count ? nb_lo + nb : 0) * KS + ks) * 64 + lane];
#pragma unroll
            for (int g = 0; g < G; ++g) af[buf][g] = *reinterpret_cast<const v4i *>(patch + base[g] + d);
        };
        auto multiply = [&](auto buf_c) {
            constexpr int buf = decltype(buf_c)::value;
#pragma unroll
            for (int g = 0; g < G; ++g) {
#pragma unroll
                for (int nb = 0; nb < NBW; ++nb) acc[g][nb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[buf][nb], af[buf][g], acc[g][nb], 0, 0, 0);
            }
        };
        typedef std::integral_constant<int, 0> b0;
        typedef std::integral_constant<int, 1> b1;
        read_step(0, b0{});
        int ks = 0;
        for (; ks + 2 <= KS; ks += 2) {
            read_step(ks + 1, b1{});
            multiply(b0{});
            if (ks + 2 < KS) read_step(ks + 2, b0{});
            multiply(b1{});
        }
        if (ks < KS) multiply(b0{});  // odd step count: the last step sits in the first set

        // ---- epilogue: 16 consecutive channels of one pixel per lane and channel block
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const int pidx = (g0 + GW * g) * 32 + r;
            const bool ok = g < ng && pidx < pixels;
            uint8_t *const row = p.out + out_tile + (size_t)(ok ? pidx : 0) * (size_t)p.ldc;
            int late = 0;
            if constexpr (late_corr) late = pixel_term(g);
#pragma unroll
            for (int nbw = 0; nbw < NBW; ++nbw) {
                const int nb = nb_lo + nbw;
                const int n = (nb_first + nb) * 32 + half * 16;
                uint32_t packed[4];
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) {
                    const int32_t x0 = acc[g][nbw][q4 * 4 + 0], x1 = acc[g][nbw][q4 * 4 + 1];
                    const int32_t x2 = acc[g][nbw][q4 * 4 + 2], x3 = acc[g][nbw][q4 * 4 + 3];
                    uint32_t o0, o1, o2, o3;
                    if constexpr (PC) {  // the padded per-channel arrays cover whole blocks
                        const int4 cm = *reinterpret_cast<const int4 *>(rq.pc_multiplier + n + q4 * 4);
                        const int4 cs = *reinterpret_cast<const int4 *>(rq.pc_shift + n + q4 * 4);
                        if constexpr (QM != 0) {
                            o0 = requant_u8_channel_fast<QM>(x0, cm.x, cs.x, rq), o1 = requant_u8_channel_fast<QM>(x1, cm.y, cs.y, rq);
                            o2 = requant_u8_channel_fast<QM>(x2, cm.z, cs.z, rq), o3 = requant_u8_channel_fast<QM>(x3, cm.w, cs.w, rq);
                        } else {
                            o0 = requant_u8_channel(x0, cm.x, cs.x, rq), o1 = requant_u8_channel(x1, cm.y, cs.y, rq);
                            o2 = requant_u8_channel(x2, cm.z, cs.z, rq), o3 = requant_u8_channel(x3, cm.w, cs.w, rq);
                        }
                    } else if constexpr (QM != 0) {
                        packed[q4] = requant4_fast<QM>(x0, x1, x2, x3, late, rq) ^ p.out_xor;
                        continue;
                    } else {
                        o0 = requant_u8_as<QM>(x0, rq), o1 = requant_u8_as<QM>(x1, rq);
                        o2 = requant_u8_as<QM>(x2, rq), o3 = requant_u8_as<QM>(x3, rq);
                    }
                    packed[q4] = pack_bytes(o0, o1, o2, o3) ^ p.out_xor;
                }
                if (ok && nb < nb_count && n < p.n) {
                    uint8_t *dst = row + n;
                    if (wide && n + 16 <= p.n) {
                        *reinterpret_cast<uint4 *>(dst) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
                    } else {
                        store_bytes_any_alignment(dst, packed, p.n - n < 16 ? p.n - n : 16);
                    }
                }
            }
        }
    }
}

constexpr size_t kLdsTwoPerCu = 80 * 1024, kLdsMax = 160 * 1024;

// LDS bytes per patch pixel: the channels and one or two chunks of slack, an odd number of 16-byte chunks in all
int conv3_pitch(int cin) { return cin + ((cin & 16) ? 32 : 16); }

size_t conv3_lds_bytes(int nb, int cin, int wo, int th) {
    const size_t ks = ((size_t)9 * cin + 31) / 32;
    const size_t head = ((size_t)nb * ks * 1024 + (size_t)nb * 128 + ks * 8 + 1023) & ~(size_t)1023;
    return head + (size_t)(th + 2) * (wo + 2) * conv3_pitch(cin);
}

// Tile height and channel blocks per workgroup for a problem.  Two workgroups per CU hide each other's staging and
// epilogue, so shapes whose LDS footprint allows that come first; among them the one that wastes the fewest rows,
// pixel-group slots and CU slots wins, two channel blocks (one patch for 64 channels) before one.
void conv3_shape(int n_img, int ho, int wo, int cin, int cout, int *th_out, int *nb_out) {
    const int n_blocks = (cout + 31) / 32;
    double best = -1;
    *th_out = 1;
    *nb_out = 1;
    for (int pass = 0; pass < 2 && best < 0; ++pass) {  // second pass: whatever fits LDS at all
        const size_t limit = pass == 0 ? kLdsTwoPerCu : kLdsMax;
        for (int nb = 1; nb <= (n_blocks >= 2 ? 2 : 1); ++nb) {
            const int parts = (n_blocks + nb - 1) / nb;
            for (int th = 1; th <= ho && th <= 32; ++th) {
                if (conv3_lds_bytes(nb, cin, wo, th) > limit) break;
                const long wgs = (long)n_img * ((ho + th - 1) / th) * parts;
                const int pixels = th * wo, groups = (pixels + 31) / 32, per_wave = (groups + 3) / 4;
                const double rows_eff = (double)ho / (((ho + th - 1) / th) * th);
                const double wave_eff = (double)pixels / (4.0 * per_wave * 32);
                const long slots = pass == 0 ? 512 : 256;
                const double fill = wgs >= slots ? (double)wgs / (((wgs + slots - 1) / slots) * slots) : (double)wgs / slots;
                // the halo rows are fetched once per tile, the weights once per workgroup
                const double traffic = (double)(th * wo * cin) / ((double)(th + 2) * (wo + 2) * cin + (double)nb * 32 * 9 * cin);
                const double score = rows_eff * wave_eff * fill * (0.6 + 0.4 * traffic) * (nb == 2 ? 1.0 : 0.8);
                if (score > best) {
                    best = score;
                    *th_out = th;
                    *nb_out = nb;
                }
            }
        }
    }
}

// G and SPLIT for a tile of `groups` pixel groups: four groups per pass where a wave has three or more to do, one
// otherwise; two-group tiles with two channel blocks spread their four (group, block) pairs over the four waves.
struct Conv3Variant {
    int g;
    bool split;
};
Conv3Variant conv3_variant(int groups, int nb) {
    Conv3Variant v;
    v.split = nb == 2 && groups <= 2;
    v.g = (groups + 3) / 4 >= 3 ? 4 : 1;
    if (v.split) v.g = 1;
    return v;
}

template <int NB>
int launch_nb(const GemmProblem &p, const Conv3Launch &L, size_t lds, hipStream_t stream) {
    const int n_blocks = (p.n + 31) / 32;
    const dim3 grid((unsigned)((L.tiles + 7) / 8 * 8), (unsigned)((n_blocks + NB - 1) / NB));
    const int rows = L.th < p.ho ? L.th : p.ho;
    const Conv3Variant variant = conv3_variant((rows * p.wo + 31) / 32, NB);
    auto launch_g = [&](auto rowsum_c, auto qm_c, auto pc_c, auto g_c, auto split_c) {
        auto kernel = conv3x3_patch_kernel<NB, decltype(rowsum_c)::value, decltype(qm_c)::value, decltype(pc_c)::value, decltype(g_c)::value,
                                           decltype(split_c)::value>;
        hipLaunchKernelGGL(kernel, grid, dim3(256), lds, stream, p, L);
        return (int)EH_OK;
    };
    auto launch_pc = [&](auto rowsum_c, auto qm_c, auto pc_c) {
        if constexpr (NB == 2) {
            if (variant.split) return launch_g(rowsum_c, qm_c, pc_c, std::integral_constant<int, 1>{}, std::true_type{});
        }
        if (variant.g == 1) return launch_g(rowsum_c, qm_c, pc_c, std::integral_constant<int, 1>{}, std::false_type{});
        return launch_g(rowsum_c, qm_c, pc_c, std::integral_constant<int, 4>{}, std::false_type{});
    };
    auto launch = [&](auto rowsum_c, auto qm_c) {
        return p.rq.pc_multiplier ? launch_pc(rowsum_c, qm_c, std::true_type{}) : launch_pc(rowsum_c, qm_c, std::false_type{});
    };
    auto with_qm = [&](auto rowsum_c) {
        if (p.rq.fast == 2) return launch(rowsum_c, std::integral_constant<int, 2>{});
        if (p.rq.fast == 1) return launch(rowsum_c, std::integral_constant<int, 1>{});
        return launch(rowsum_c, std::integral_constant<int, 0>{});
    };
    const int rc = p.zw != 0 ? with_qm(std::true_type{}) : with_qm(std::false_type{});
    if (rc) return rc;
    EH_HIP(hipGetLastError());
    return EH_OK;
}

}  // namespace

// 3x3 taps at dilation 1 and stride 1 over all of the input's channels, which come in whole 16-byte chunks, on an
// output wide enough that a tile of rows fills the waves, and a patch of three rows that fits LDS beside the weights.
bool conv3x3_patch_applies(int32_t cin_group, int32_t pixel_stride, int32_t wo, int32_t ho) {
    if (cin_group != pixel_stride || (cin_group & 15) != 0 || cin_group > 128) return false;
    if (wo < 8 || (long)wo * ho < 128) return false;
    return conv3_lds_bytes(1, cin_group, wo, 1) <= kLdsMax;
}

// Allows every variant of the kernel its dynamic LDS beyond 64 KiB on the current device.  Done once per device when the
// library is initialised on it, so that a launch (which may sit in a capture or in a caller that must not meet the
// driver) is a launch and nothing else.
static std::atomic<bool> g_conv3_prepared{false};

int conv3x3_patch_prepare() {
    int rc = EH_OK;
    auto raise = [&](auto kernel) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsMax);
        if (e != hipSuccess && rc == EH_OK) rc = hip_fail(e, "hipFuncSetAttribute(conv3x3_patch_kernel)");
    };
    auto each_pc = [&](auto nb_c, auto rowsum_c, auto qm_c) {
        constexpr int NB = decltype(nb_c)::value;
        constexpr bool RS = decltype(rowsum_c)::value;
        constexpr int QM = decltype(qm_c)::value;
        raise(conv3x3_patch_kernel<NB, RS, QM, false, 4, false>);
        raise(conv3x3_patch_kernel<NB, RS, QM, true, 4, false>);
        raise(conv3x3_patch_kernel<NB, RS, QM, false, 1, false>);
        raise(conv3x3_patch_kernel<NB, RS, QM, true, 1, false>);
        if constexpr (NB == 2) {
            raise(conv3x3_patch_kernel<NB, RS, QM, false, 1, true>);
            raise(conv3x3_patch_kernel<NB, RS, QM, true, 1, true>);
        }
    };
    auto each_qm = [&](auto nb_c, auto rowsum_c) {
        each_pc(nb_c, rowsum_c, std::integral_constant<int, 0>{});
        each_pc(nb_c, rowsum_c, std::integral_constant<int, 1>{});
        each_pc(nb_c, rowsum_c, std::integral_constant<int, 2>{});
    };
    auto each_rowsum = [&](auto nb_c) {
        each_qm(nb_c, std::false_type{});
        each_qm(nb_c, std::true_type{});
    };
    each_rowsum(std::integral_constant<int, 1>{});
    each_rowsum(std::integral_constant<int, 2>{});
    if (rc == EH_OK) g_conv3_prepared.store(true, std::memory_order_release);
    return rc;
}

int launch_conv3x3_patch(const GemmProblem &p, hipStream_t stream) {
    EH_REQUIRE(p.k == 9 * p.cin && (p.cin & 15) == 0 && p.k_pad == (p.k + 31) / 32 * 32 && p.stride_h == 1 && p.stride_w == 1,
               "conv3x3: unsupported problem (k %d, cin %d)", p.k, p.cin);
    // the kernel addresses the output as one dense image per input image: no window, offset or stride on the output side
    EH_REQUIRE(p.out_sy == 1 && p.out_sx == 1 && p.out_y0 == 0 && p.out_x0 == 0 && p.out_h == p.ho && p.out_w == p.wo,
               "conv3x3: the output must be the whole dense image (window %d x %d at %d,%d step %d,%d for %d x %d)", p.out_h, p.out_w,
               p.out_y0, p.out_x0, p.out_sy, p.out_sx, p.ho, p.wo);
    EH_REQUIRE((reinterpret_cast<uintptr_t>(p.a) & 15) == 0, "conv3x3: input pointer is not aligned to 16 bytes");
    const int n_img = p.m / (p.ho * p.wo);
    int th = 1, nb = 1;
    conv3_shape(n_img, p.ho, p.wo, p.cin, p.n, &th, &nb);
    Conv3Launch L;
    L.th = th;
    L.tiles_per_image = (p.ho + th - 1) / th;
    L.tiles = n_img * L.tiles_per_image;
    L.ksteps = p.k_pad / 32;
    L.pitch = conv3_pitch(p.cin);
    L.pc = p.wo + 2;
    L.div_pch = make_fastdiv((uint32_t)(L.pitch >> 4));
    L.div_pc = make_fastdiv((uint32_t)L.pc);
    L.div_wo = make_fastdiv((uint32_t)p.wo);
    L.div_tiles = make_fastdiv((uint32_t)L.tiles_per_image);
    const size_t lds = conv3_lds_bytes(nb, p.cin, p.wo, th);
    EH_REQUIRE(lds <= kLdsMax, "conv3x3: %zu bytes of LDS", lds);
    if (!g_conv3_prepared.load(std::memory_order_acquire)) {  // a caller that never went through eh_init
        const int rc = conv3x3_patch_prepare();
        if (rc) return rc;
    }
    return nb == 2 ? launch_nb<2>(p, L, lds, stream) : launch_nb<1>(p, L, lds, stream);
}

}  // namespace eh
