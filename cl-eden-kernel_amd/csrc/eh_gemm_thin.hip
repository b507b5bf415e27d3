// uint8 GEMM kernel for one-tap problems (1x1 convolutions, fully-connected layers)
// that are short of work for the tiled kernels: at most 64 reduction bytes
// (pointwise expansions such as 24 -> 144), or a small pixel count (the late
// layers of an image network, classifier heads).
//
// Such layers are bound by memory, by the requantization arithmetic or by latency,
// not by the matrix cores.  A workgroup copies the weights of its channel range
// (packed in MFMA fragment order, 1 KiB per 32-channel block and 32-byte step) and
// their bias into LDS once; each of its waves then walks 32-pixel blocks: every lane
// fetches 16 reduction bytes of its pixel per step straight into the 32x32x32 MFMA
// fragment layout (the bytes of a wave are one contiguous span when the pixels are),
// with the next block's bytes requested before the current block's arithmetic, and
// finishes the range's channel blocks against the weights in LDS.  The activations
// are read once per channel range, the weights once per workgroup.
// The weight fragment is the row operand and its rows are permuted within a
// 32-channel block (see packed_b_offset), so a lane ends up with 16 consecutive
// output channels of its pixel: requantize, pack, one 16-byte store.
#include <type_traits>

#include <atomic>

#include "eh_internal.h"

namespace eh {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

namespace {

typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t u32x2_a4 __attribute__((ext_vector_type(2), aligned(4)));

// NBU: channel blocks a wave finishes per pass; KU: reduction steps whose loads are in flight together.
// Grid: x = workgroups along the pixel rows (each wave walks 32-row blocks with stride gridDim.x * 4),
// y = channel ranges of `nbw` blocks.
// QM: how results are requantized.  0: the two-step order (one pair, or one per channel read from global memory);
// 1: the single-shift form with the requant's one pair; 2: the single-shift form with one pair per channel, whose
// multiplier, shift and rounding term sit in LDS beside the bias.
// Output staging (stage_pitch != 0; launches whose workgroups own whole pixels of a densely stored output, no residual):
// a lane's sixteen bytes go to a per-wave LDS image of the block's 32 pixels first, and the wave then writes that
// image out as one contiguous span, 16 bytes per lane.  A pixel block's output is contiguous in memory (32 x ldc
// bytes), but a lane holds 16 channels of one pixel, so storing from the accumulator layout makes every store
// instruction touch 32 separate sectors of 32 bytes; from the image it writes whole 128-byte lines.
struct ThinStage {
    int32_t pitch;     // LDS bytes per pixel of the image (an odd number of 16-byte chunks), 0: store directly
    int32_t offset;    // byte offset of the four waves' images in dynamic LDS
    FastDiv div_cpp;   // chunks of 16 bytes per pixel: ldc / 16
    // 1: pixel m of the GEMM reads at m * cin and writes at m * ldc (stride 1, no offsets, dense output), every factor
    // below 2^24 and every product below 2^32, so a lane finds its pixel with two full-rate multiplies instead of two
    // divisions and a dozen 32- and 64-bit multiplies (which issue at a quarter of the rate)
    int32_t linear;
};

// one problem, or (BATCHED) up to eight equally shaped ones along grid z
__device__ __forceinline__ const GemmProblem &problem_of(const GemmProblem &one) { return one; }
__device__ __forceinline__ const GemmProblem &problem_of(const GemmBatch &batch) { return batch.p[blockIdx.z]; }

template <int NBU, int KU, bool ROWSUM, int QM, bool RES, bool BATCHED = false>
__global__ __launch_bounds__(256) void direct_gemm_kernel(const std::conditional_t<BATCHED, GemmBatch, GemmProblem> arg, const int n_blocks,
                                                          const int ksteps, const int nbw, const int row_blocks, const ThinStage stage) {
    // BATCHED: equally shaped problems of one operator (the output phases of a transposed convolution whose kernel is its
    // stride) that differ in their weights and in where their outputs go.  (A kernel of its own: indexing the argument
    // costs the single problem 2 - 3 %.)
    const GemmProblem &p = problem_of(arg);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 31, half = lane >> 5;
    const int plane = p.ho * p.wo;
    const int nb_first = blockIdx.y * nbw;
    const int nb_count = n_blocks - nb_first < nbw ? n_blocks - nb_first : nbw;  // blocks of this range that exist

    // this range's weights (fragment order: 1 KiB per block and step) and bias live in LDS, copied once per workgroup
    extern __shared__ __align__(16) uint8_t lds_raw[];
    v4i *b_s = reinterpret_cast<v4i *>(lds_raw);                                  // [nbw][ksteps][64 lanes]
    int32_t *bias_s = reinterpret_cast<int32_t *>(lds_raw + (size_t)nbw * ksteps * 1024);  // [nbw * 32]
    // fused residual add: the rescaled value of every possible residual byte and of every possible result byte, so that
    // an output costs two lookups and one rescaling instead of three rescalings
    // per-channel single-shift tables, only with QM == 2: multiplier, right shift - 1, high word of the rounding term
    int32_t *pcm_s = bias_s + nbw * 32, *pcf_s = pcm_s + nbw * 32, *pch_s = pcf_s + nbw * 32;
    int32_t *add_a_s = bias_s + (QM == 2 ? 4 : 1) * nbw * 32, *add_b_s = add_a_s + 256;  // [256] each, only with RES
    auto stage_weights = [&]() {
        const v4i *src = reinterpret_cast<const v4i *>(p.b) + (size_t)nb_first * ksteps * 64;
        const int pieces = nb_count * ksteps * 64;
        for (int i = threadIdx.x; i < pieces; i += 256) b_s[i] = src[i];
        for (int i = threadIdx.x; i < nb_count * 32; i += 256) bias_s[i] = p.bias[nb_first * 32 + i];
        if constexpr (QM == 2) {
            // rounding term 2^30 + (1 + 2 zp_out) 2^(30 + rs) for rs >= 2: low word 2^30, high word (1 + 2 zp_out) 2^(rs - 2)
            for (int i = threadIdx.x; i < nb_count * 32; i += 256) {
                const int32_t rs = -p.rq.pc_shift[nb_first * 32 + i];
                pcm_s[i] = p.rq.pc_multiplier[nb_first * 32 + i];
                pcf_s[i] = rs - 1;
                pch_s[i] = channel_table_pos_hi(p.rq.zp_out, rs);
            }
        }
        if constexpr (RES) {
            const int byte = threadIdx.x;  // 256 threads, 256 byte values
            add_a_s[byte] = mul_round_shift((int32_t)((uint32_t)(byte - p.radd.zp_a) << p.radd.left_shift), p.radd.mult_a, p.radd.rs_a);
            add_b_s[byte] = mul_round_shift((int32_t)((uint32_t)(byte - p.radd.zp_b) << p.radd.left_shift), p.radd.mult_b, p.radd.rs_b);
        }
        __syncthreads();
    };
    // add_word with the two tables (the same arithmetic: the tables hold what add_one computes first)
    auto add_word_lut = [&](uint32_t a, uint32_t b) {
        uint32_t out = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int32_t sum = add_a_s[(a >> (8 * i)) & 255u] + add_b_s[(b >> (8 * i)) & 255u];
            int32_t v = mul_round_shift(sum, p.radd.mult_out, p.radd.rs_out) + p.radd.zp_out;
            v = v < p.radd.act_min ? p.radd.act_min : v;
            v = v > p.radd.act_max ? p.radd.act_max : v;
            out |= (uint32_t)v << (8 * i);
        }
        return out;
    };

    const RequantDev rq = p.rq;
    const bool wide = (p.ldc & 3) == 0 && ((reinterpret_cast<uintptr_t>(p.out) & 3) == 0);  // dword-aligned rows: vector stores
    // XCD x (workgroups x, x + 8, ...: gridDim.x is a multiple of 8) owns the x-th contiguous eighth of the row blocks
    const int rb_per_xcd = (row_blocks + 7) >> 3;
    const int rb_first = (int)(blockIdx.x & 7u) * rb_per_xcd + (int)(blockIdx.x >> 3) * 4 + wave;
    const int rb_end = ((int)(blockIdx.x & 7u) + 1) * rb_per_xcd < row_blocks ? ((int)(blockIdx.x & 7u) + 1) * rb_per_xcd : row_blocks;
    const int rb_stride = (int)(gridDim.x >> 3) * 4;
    constexpr bool SINGLE = KU < 4;  // the whole reduction is one group of KU steps (the launcher guarantees ksteps <= KU)

    // where the lane's pixel of row block `rb` reads and writes
    auto locate = [&](int rb, bool &ok, size_t &in_off, size_t &out_off) {
        const int m = rb * 32 + r;
        ok = rb < rb_end && m < p.m;
        in_off = 0;
        out_off = 0;
        if (ok && stage.linear) {
            in_off = (size_t)(__umul24((uint32_t)m, (uint32_t)p.cin) + (uint32_t)p.a_offset + (uint32_t)half * 16u);
            out_off = (size_t)__umul24((uint32_t)m, (uint32_t)p.ldc);
        } else if (ok) {
            const int img = (int)fastdiv((uint32_t)m, p.div_plane), rem = m - img * plane;
            const int oy = (int)fastdiv((uint32_t)rem, p.div_wo), ox = rem - oy * p.wo;
            in_off = ((size_t)(img * p.h + oy * p.stride_h + p.y_base) * p.w + (ox * p.stride_w + p.x_base)) * (size_t)p.cin +
                     (size_t)p.a_offset + half * 16;
            out_off = (((size_t)img * p.out_h + (oy * p.out_sy + p.out_y0)) * p.out_w + (ox * p.out_sx + p.out_x0)) * (size_t)p.ldc;
        }
    };
    // 16 reduction bytes of step ks; bytes past K read as the byte that the sign flip turns into 0
    auto load_a = [&](bool ok, size_t in_off, int ks, uint2 &lo, uint2 &hi) {
        const int kb = ks * 32 + half * 16;
        lo = make_uint2(p.a_xor, p.a_xor);
        hi = lo;
        if (ok && kb < p.k) lo = *reinterpret_cast<const uint2 *>(p.a + in_off + ks * 32);
        if (ok && kb + 8 < p.k) hi = *reinterpret_cast<const uint2 *>(p.a + in_off + ks * 32 + 8);
    };
    auto to_fragment = [&](uint2 lo, uint2 hi, int &rowsum) {
        v4i af;
        af.x = (int)(lo.x ^ p.a_xor);
        af.y = (int)(lo.y ^ p.a_xor);
        af.z = (int)(hi.x ^ p.a_xor);
        af.w = (int)(hi.y ^ p.a_xor);
        if constexpr (ROWSUM) {
            rowsum = __builtin_amdgcn_sdot4(af.x, 0x01010101, rowsum, false);
            rowsum = __builtin_amdgcn_sdot4(af.y, 0x01010101, rowsum, false);
            rowsum = __builtin_amdgcn_sdot4(af.z, 0x01010101, rowsum, false);
            rowsum = __builtin_amdgcn_sdot4(af.w, 0x01010101, rowsum, false);
        }
        return af;
    };
    // The accumulators start from the folded bias (plus `extra`, the pixel's row-sum term where it is known before the
    // products): the matrix instruction adds to them, so the epilogue has no additions left to do.
    constexpr bool late_corr = ROWSUM && QM == 1;
    auto start_block = [&](int nb_local, int extra = 0) {
        const int32_t *bsrc = bias_s + nb_local * 32 + half * 16;
        v16i acc;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int4 bb = *reinterpret_cast<const int4 *>(bsrc + g * 4);
            acc[g * 4 + 0] = bb.x + extra;
            acc[g * 4 + 1] = bb.y + extra;
            acc[g * 4 + 2] = bb.z + extra;
            acc[g * 4 + 3] = bb.w + extra;
        }
        return acc;
    };
    // 16 accumulators of one channel block (bias included) -> 16 output bytes of the lane's pixel; `ncorr` is what
    // is still to be added to each
    auto finish_block = [&](const v16i &acc, int nb_local, int ncorr, bool ok, size_t out_off) {
        const int n = (nb_first + nb_local) * 32 + half * 16;  // this lane's 16 consecutive channels
        uint32_t packed[4];
        auto quantize = [&](auto mode_c) {
            constexpr int mode = decltype(mode_c)::value;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                uint32_t o0, o1, o2, o3;
                if constexpr (QM == 2) {
                    const int tab = nb_local * 32 + half * 16 + g * 4;
                    const int4 cm = *reinterpret_cast<const int4 *>(pcm_s + tab);
                    const int4 cf = *reinterpret_cast<const int4 *>(pcf_s + tab);
                    const int4 ch = *reinterpret_cast<const int4 *>(pch_s + tab);
                    o0 = requant_u8_channel_table<mode>(acc[g * 4 + 0] + ncorr, cm.x, cf.x, ch.x, rq);
                    o1 = requant_u8_channel_table<mode>(acc[g * 4 + 1] + ncorr, cm.y, cf.y, ch.y, rq);
                    o2 = requant_u8_channel_table<mode>(acc[g * 4 + 2] + ncorr, cm.z, cf.z, ch.z, rq);
                    o3 = requant_u8_channel_table<mode>(acc[g * 4 + 3] + ncorr, cm.w, cf.w, ch.w, rq);
                } else if (mode == 0 && rq.pc_multiplier) {  // per-channel parameters (the padded arrays cover whole blocks)
                    const int4 cm = *reinterpret_cast<const int4 *>(rq.pc_multiplier + n + g * 4);
                    const int4 cs = *reinterpret_cast<const int4 *>(rq.pc_shift + n + g * 4);
                    o0 = requant_u8_channel(acc[g * 4 + 0] + ncorr, cm.x, cs.x, rq);
                    o1 = requant_u8_channel(acc[g * 4 + 1] + ncorr, cm.y, cs.y, rq);
                    o2 = requant_u8_channel(acc[g * 4 + 2] + ncorr, cm.z, cs.z, rq);
                    o3 = requant_u8_channel(acc[g * 4 + 3] + ncorr, cm.w, cs.w, rq);
                } else if constexpr (mode != 0) {
                    packed[g] = requant4_fast<mode>(acc[g * 4 + 0], acc[g * 4 + 1], acc[g * 4 + 2], acc[g * 4 + 3], ncorr, rq) ^ p.out_xor;
                    continue;
                } else {
                    o0 = requant_u8_as<mode>(acc[g * 4 + 0] + ncorr, rq);
                    o1 = requant_u8_as<mode>(acc[g * 4 + 1] + ncorr, rq);
                    o2 = requant_u8_as<mode>(acc[g * 4 + 2] + ncorr, rq);
                    o3 = requant_u8_as<mode>(acc[g * 4 + 3] + ncorr, rq);
                }
                packed[g] = pack_bytes(o0, o1, o2, o3) ^ p.out_xor;
            }
        };
        if constexpr (QM == 0)
            quantize(std::integral_constant<int, 0>{});
        else if (rq.fast == 2)
            quantize(std::integral_constant<int, 2>{});
        else
            quantize(std::integral_constant<int, 1>{});
        if constexpr (!RES) {
            if (stage.pitch) {  // (every channel block is whole here: the launcher asks for n % 16 == 0)
                if (n < p.n)
                    *reinterpret_cast<uint4 *>(lds_raw + stage.offset + (wave * 32 + r) * stage.pitch + n) =
                        make_uint4(packed[0], packed[1], packed[2], packed[3]);
                return;
            }
        }
        if (!ok || n >= p.n) return;
        uint8_t *dst = p.out + out_off + n;
        const int cnt = p.n - n;
        if constexpr (RES) {  // out = add(residual, result); the residual tensor is addressed like the output
            const uint8_t *res = p.residual + out_off + n;
            if (wide && (cnt >= 16 || cnt == 8)) {
                // (a block's second half may hold eight channels only, as with 24 or 56 of them: its upper words are
                // computed from zeros and never stored)
                const u32x2_a4 lo = *reinterpret_cast<const u32x2_a4 *>(res);
                u32x2_a4 hi = {0u, 0u};
                if (cnt >= 16) hi = *reinterpret_cast<const u32x2_a4 *>(res + 8);
                packed[0] = add_word_lut(lo.x, packed[0]);
                packed[1] = add_word_lut(lo.y, packed[1]);
                packed[2] = add_word_lut(hi.x, packed[2]);
                packed[3] = add_word_lut(hi.y, packed[3]);
            } else {
                const int c = cnt < 16 ? cnt : 16;
                for (int t = 0; t < c; ++t) {
                    const uint32_t v = add_one(res[t], (packed[t >> 2] >> (8 * (t & 3))) & 255u, p.radd);
                    packed[t >> 2] = (packed[t >> 2] & ~(255u << (8 * (t & 3)))) | (v << (8 * (t & 3)));
                }
            }
        }
        if (wide && cnt >= 16) {
            *reinterpret_cast<u32x4_a4 *>(dst) = u32x4_a4{packed[0], packed[1], packed[2], packed[3]};
        } else if (wide && cnt == 8) {
            *reinterpret_cast<u32x2_a4 *>(dst) = u32x2_a4{packed[0], packed[1]};
        } else {
            // (whole chunks of rows that start at odd addresses: dwords at byte addresses; written out here because the
            // shared helper's per-dword tests cost the aligned path 2.5 % through register allocation)
            if (cnt >= 16) {
#pragma unroll
                for (int g = 0; g < 4; ++g) *reinterpret_cast<u32_any_alignment *>(dst + 4 * g) = packed[g];
            } else {
                for (int t = 0; t < cnt; ++t) dst[t] = (uint8_t)(packed[t >> 2] >> (8 * (t & 3)));
            }
        }
    };

    // writes the wave's staged image of row block `rb` out as one contiguous span
    auto flush_stage = [&](int rb) {
        const int first = rb * 32;
        const int pixels = p.m - first < 32 ? p.m - first : 32;
        const int cpp = p.ldc >> 4, chunks = pixels * cpp;
        const uint8_t *img = lds_raw + stage.offset + wave * 32 * stage.pitch;
        uint8_t *dst = p.out + (size_t)first * (size_t)p.ldc;
        for (int c = lane; c < chunks; c += 64) {
            const int px = (int)fastdiv((uint32_t)c, stage.div_cpp), col = c - px * cpp;
            *reinterpret_cast<uint4 *>(dst + (size_t)c * 16) = *reinterpret_cast<const uint4 *>(img + px * stage.pitch + col * 16);
        }
    };

    if constexpr (SINGLE) {
        // the pixel block's reduction bytes sit in registers for all of its channel blocks; the next
        // block's bytes are requested before this one's arithmetic starts
        bool ok, ok_next;
        size_t in_off, out_off, in_next, out_next;
        uint2 lo[KU], hi[KU], lo_next[KU], hi_next[KU];
        int rb = rb_first;
        locate(rb, ok, in_off, out_off);
#pragma unroll
        for (int t = 0; t < KU; ++t) load_a(ok, in_off, t, lo[t], hi[t]);
        stage_weights();  // after the first activation loads are on their way: the two latencies overlap
        for (; rb < rb_end; rb += rb_stride) {
            locate(rb + rb_stride, ok_next, in_next, out_next);
#pragma unroll
            for (int t = 0; t < KU; ++t) load_a(ok_next, in_next, t, lo_next[t], hi_next[t]);
            v4i af[KU];
            int rowsum = 0;
#pragma unroll
            for (int t = 0; t < KU; ++t) af[t] = to_fragment(lo[t], hi[t], rowsum);
            int ncorr = 0;
            if constexpr (ROWSUM) {
                rowsum += __shfl_xor(rowsum, 32);  // the other half of this pixel's reduction bytes
                ncorr = -p.zw * rowsum;
            }
            for (int nb0 = 0; nb0 < nb_count; nb0 += NBU) {
                v4i bf[NBU][KU];
#pragma unroll
                for (int u = 0; u < NBU; ++u) {
                    const int nb = nb0 + u < nb_count ? nb0 + u : nb_count - 1;
#pragma unroll
                    for (int t = 0; t < KU; ++t) bf[u][t] = b_s[(nb * ksteps + (t < ksteps ? t : ksteps - 1)) * 64 + lane];
                }
#pragma unroll
                for (int u = 0; u < NBU; ++u) {
                    if (nb0 + u >= nb_count) break;
                    // (the single-shift forms take the pixel's term inside their rounding term: nothing to add per accumulator)
                    v16i acc = late_corr ? start_block(nb0 + u) : start_block(nb0 + u, ncorr);
#pragma unroll
                    for (int t = 0; t < KU; ++t) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[u][t], af[t], acc, 0, 0, 0);
                    finish_block(acc, nb0 + u, late_corr ? ncorr : 0, ok, out_off);
                }
            }
            if constexpr (!RES) {
                if (stage.pitch) flush_stage(rb);
            }
            ok = ok_next;
            in_off = in_next;
            out_off = out_next;
#pragma unroll
            for (int t = 0; t < KU; ++t) {
                lo[t] = lo_next[t];
                hi[t] = hi_next[t];
            }
        }
    } else {
        stage_weights();
        for (int rb = rb_first; rb < rb_end; rb += rb_stride) {
            bool ok;
            size_t in_off, out_off;
            locate(rb, ok, in_off, out_off);
            for (int nb0 = 0; nb0 < nb_count; nb0 += NBU) {
                v16i acc[NBU];
#pragma unroll
                for (int u = 0; u < NBU; ++u) acc[u] = start_block(nb0 + u < nb_count ? nb0 + u : nb_count - 1, 0);
                int rowsum = 0;
                for (int ks0 = 0; ks0 < ksteps; ks0 += KU) {
                    // steps past the last one read bytes that flip to 0, so they multiply whatever weights they re-read by zero
                    uint2 lo[KU], hi[KU];
#pragma unroll
                    for (int t = 0; t < KU; ++t) load_a(ok, in_off, ks0 + t, lo[t], hi[t]);
#pragma unroll
                    for (int t = 0; t < KU; ++t) {
                        const v4i af = to_fragment(lo[t], hi[t], rowsum);
                        const int ks = ks0 + t < ksteps ? ks0 + t : ksteps - 1;
#pragma unroll
                        for (int u = 0; u < NBU; ++u) {
                            const int nb = nb0 + u < nb_count ? nb0 + u : nb_count - 1;
                            acc[u] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b_s[(nb * ksteps + ks) * 64 + lane], af, acc[u], 0, 0, 0);
                        }
                    }
                }
                int ncorr = 0;
                if constexpr (ROWSUM) {
                    rowsum += __shfl_xor(rowsum, 32);
                    ncorr = -p.zw * rowsum;
                }
#pragma unroll
                for (int u = 0; u < NBU; ++u) {
                    if (nb0 + u >= nb_count) break;
                    finish_block(acc[u], nb0 + u, ncorr, ok, out_off);
                }
            }
            if constexpr (!RES) {
                if (stage.pitch) flush_stage(rb);
            }
        }
    }
}

template <int NBU, int KU>
int launch_nbu(const GemmProblem *ps, int count, hipStream_t stream) {
    const GemmProblem &p = ps[0];
    GemmBatch batch;
    for (int i = 0; i < count; ++i) batch.p[i] = ps[i];
    const int n_blocks = (p.n + 31) / 32, ksteps = p.k_pad / 32;
    const int row_blocks = (p.m + 31) / 32;
    // Channel ranges: as few as the LDS budget for the weights allows (32 KiB, so that several workgroups share a CU),
    // more when the pixel rows alone do not give every SIMD a few waves.
    const int groups_total = (n_blocks + NBU - 1) / NBU;
    int nbw_max = (32 / ksteps) / NBU * NBU;
    if (nbw_max < NBU) nbw_max = NBU;
    int ranges = (n_blocks + nbw_max - 1) / nbw_max;
    const bool dense_out = p.out_sy == 1 && p.out_sx == 1 && p.out_y0 == 0 && p.out_x0 == 0 && p.out_h == p.ho && p.out_w == p.wo;
    const bool stageable = !p.residual && p.n == p.ldc && (p.n & 15) == 0 && p.n <= 256 && dense_out &&
                           (reinterpret_cast<uintptr_t>(p.out) & 15) == 0;
    while (ranges < groups_total && (long)row_blocks * ranges < 4096) ++ranges;
    const int nbw = (groups_total + ranges - 1) / ranges * NBU;
    ranges = (n_blocks + nbw - 1) / nbw;
    const bool pc_fast = p.rq.fast && p.rq.pc_multiplier;
    const size_t lds = (size_t)nbw * ksteps * 1024 + (size_t)nbw * 32 * sizeof(int32_t) * (pc_fast ? 4 : 1) +
                       (p.residual ? 2 * 256 * sizeof(int32_t) : 0);
    EH_REQUIRE(lds <= 64 * 1024, "igemm_thin: %zu bytes of LDS for the weights", lds);
    // Staged output where a workgroup owns whole, densely stored pixels of at most 256 bytes (wider pixels already fill
    // whole lines per store, and the images would crowd the CU's LDS)
    ThinStage stage{};
    if (ranges == 1 && stageable) {
        const int cpp = p.ldc / 16;
        stage.pitch = (cpp | 1) * 16;
        stage.offset = (int32_t)((lds + 15) / 16 * 16);
        stage.div_cpp = make_fastdiv((uint32_t)cpp);
        if ((size_t)stage.offset + 4u * 32u * stage.pitch > 64 * 1024) stage = ThinStage{};
    }
    const size_t lds_all = stage.pitch ? (size_t)stage.offset + 4u * 32u * stage.pitch : lds;
    {
        // (a batch's problems may start at different channels of the pixel: none starts beyond its end)
        const long reach_in = (long)p.m * p.cin + p.cin + 16, reach_out = (long)p.m * p.ldc;
        stage.linear = dense_out && p.stride_h == 1 && p.stride_w == 1 && p.y_base == 0 && p.x_base == 0 && p.h == p.ho && p.w == p.wo &&
                       p.a_offset >= 0 && p.m < (1 << 24) && p.cin < (1 << 24) && p.ldc < (1 << 24) && reach_in < (1l << 32) &&
                       reach_out < (1l << 32);
    }
    // row sums, the single-shift requantization and the fused residual add are compile-time variants: a launch pays for
    // none of the code it does not use
    auto launch = [&](auto rowsum_c, auto qm_c, auto res_c) {
        constexpr bool RS = decltype(rowsum_c)::value, RES = decltype(res_c)::value;
        constexpr int QM = decltype(qm_c)::value;
        const void *kernel = count > 1 ? reinterpret_cast<const void *>(direct_gemm_kernel<NBU, KU, RS, QM, false, true>)
                                       : reinterpret_cast<const void *>(direct_gemm_kernel<NBU, KU, RS, QM, RES, false>);
        // The grid is persistent: as many workgroups as the device holds at once with this variant's registers and
        // this launch's LDS (a wave has one pixel block in flight, so the bytes in flight grow with the waves), and
        // at least four per CU.  The answer is kept per KiB of LDS.
        static std::atomic<int> resident[65];
        const size_t slot = (lds_all + 1023) / 1024;
        int per_cu = resident[slot].load(std::memory_order_relaxed);
        if (per_cu == 0) {
            int n = 0;
            if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, 256, lds_all) != hipSuccess || n < 1) n = 4;
            per_cu = n < 4 ? 4 : (n > 8 ? 8 : n);
            resident[slot].store(per_cu, std::memory_order_relaxed);
        }
        int row_wgs = ((row_blocks + 7) / 8 + 3) / 4 * 8;   // a multiple of 8: every XCD walks its own eighth of the row blocks
        const int wg_target = 256 * per_cu / (ranges * count) > 8 ? 256 * per_cu / (ranges * count) / 8 * 8 : 8;
        if (row_wgs > wg_target) row_wgs = wg_target;
        if (count > 1)
            hipLaunchKernelGGL((direct_gemm_kernel<NBU, KU, RS, QM, false, true>), dim3(row_wgs, ranges, count), dim3(256), lds_all, stream, batch, n_blocks,
                               ksteps, nbw, row_blocks, stage);
        else
            hipLaunchKernelGGL((direct_gemm_kernel<NBU, KU, RS, QM, RES, false>), dim3(row_wgs, ranges), dim3(256), lds_all, stream, p, n_blocks, ksteps, nbw,
                               row_blocks, stage);
    };
    auto with_res = [&](auto rowsum_c, auto qm_c) {
        if (p.residual)
            launch(rowsum_c, qm_c, std::true_type{});
        else
            launch(rowsum_c, qm_c, std::false_type{});
    };
    auto with_qm = [&](auto rowsum_c) {
        if (pc_fast)
            with_res(rowsum_c, std::integral_constant<int, 2>{});
        else if (p.rq.fast)
            with_res(rowsum_c, std::integral_constant<int, 1>{});
        else
            with_res(rowsum_c, std::integral_constant<int, 0>{});
    };
    if (p.zw != 0)
        with_qm(std::true_type{});
    else
        with_qm(std::false_type{});
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

int launch_igemm_thin(const GemmProblem *ps, int count, hipStream_t stream) {
    const GemmProblem &p = ps[0];
    EH_REQUIRE(count >= 1 && count <= GemmBatch::MAX, "igemm_thin: batch of %d", count);
    for (int i = 1; i < count; ++i)
        EH_REQUIRE(ps[i].m == p.m && ps[i].n == p.n && ps[i].k == p.k && ps[i].k_pad == p.k_pad && ps[i].cin == p.cin && ps[i].ldc == p.ldc && ps[i].zw == p.zw &&
                       ps[i].residual == nullptr && p.residual == nullptr && ps[i].rq.fast == p.rq.fast &&
                       (ps[i].rq.pc_multiplier != nullptr) == (p.rq.pc_multiplier != nullptr) && ps[i].h == p.h && ps[i].w == p.w && ps[i].ho == p.ho &&
                       ps[i].wo == p.wo && ps[i].stride_h == p.stride_h && ps[i].stride_w == p.stride_w && ps[i].out_sy == p.out_sy && ps[i].out_sx == p.out_sx &&
                       ps[i].out_h == p.out_h && ps[i].out_w == p.out_w,
                   "igemm_thin: a batch must hold equally shaped problems");
    EH_REQUIRE(p.k_pad % 32 == 0 && p.k_pad >= p.k, "igemm_thin: padded reduction length %d", p.k_pad);
    EH_REQUIRE((p.k & 7) == 0 && (p.cin & 7) == 0 && (reinterpret_cast<uintptr_t>(p.a) & 7) == 0,
               "igemm_thin: rows must start on 8-byte boundaries");
    const int n_blocks = (p.n + 31) / 32;
    if (p.k_pad == 32) {
        if (n_blocks == 1) return launch_nbu<1, 1>(ps, count, stream);
        if (n_blocks == 2) return launch_nbu<2, 1>(ps, count, stream);
        return launch_nbu<4, 1>(ps, count, stream);
    }
    if (p.k_pad == 64) {
        if (n_blocks == 1) return launch_nbu<1, 2>(ps, count, stream);
        if (n_blocks == 2) return launch_nbu<2, 2>(ps, count, stream);
        return launch_nbu<4, 2>(ps, count, stream);
    }
    if (p.k_pad <= 192) {  // one group of six steps: a row block's loads leave together
        if (n_blocks == 1) return launch_nbu<1, 6>(ps, count, stream);
        return launch_nbu<2, 6>(ps, count, stream);
    }
    if (n_blocks == 1) return launch_nbu<1, 4>(ps, count, stream);
    return launch_nbu<2, 4>(ps, count, stream);
}

}  // namespace eh
