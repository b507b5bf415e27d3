// Pointwise expansion + depthwise 3x3 as ONE launch (gfx950): the MobileNet-style block "1x1 convolution to C expanded
// channels, activation, requantization to uint8; then a 3x3 depthwise convolution over that tensor" without the
// expanded tensor ever leaving the CU.
//
// The reference runs the two operators one after the other on its queue (gpu/gpu_op_executor.cc:56-103:
// CLConvolution -> quantizedGemmBlocked writes the expanded tensor, CLDepthwiseConvolution ->
// depthwise_conv_3x3s2_pad_merge reads it back, cl_kernels/DepthwiseconvolutionKernels.cpp:1964-2083); at the block of
// BASELINE configs[2] the expanded tensor is 14.45 MB written and read again against 2.4 MB of input and 3.6 MB of
// output.  Here a workgroup owns a tile of TH x TW output pixels of one image:
//   0. the input pixels under the tile's windows ((TH - 1) * S + 3 rows by (TW - 1) * S + 3 columns, a few KB) are copied
//      to LDS with contiguous loads, beside the pointwise weights and bias;
//   1. the expanded pixels are computed by the matrix cores (one 32x32x32 int8 MFMA per 32 pixels and 32 channels; the
//      (pixel block, channel block) pairs are dealt out evenly over the four waves), requantized exactly as the
//      pointwise operator does it and written as uint8 into an LDS image [row][column][channel]; pixels outside the
//      image are written as the depthwise operator's input zero point, which is what its padding reads;
//   2. after one barrier the threads compute the depthwise outputs from that image, four horizontally adjacent output
//      pixels of four channels per thread, with the arithmetic of the stand-alone depthwise kernel (8-bit dot products,
//      signed or unsigned form), and store them.
// The rows and columns two neighbouring workgroups both need (the halo) are computed twice; nothing else is.  Tiles are
// cut in both directions because the halo of a stride-2 window costs (2 TH + 1)(2 TW + 1) / (4 TH TW): 1.53 for one full
// row of 28 outputs, 1.21 for 4 x 7.
// A depthwise channel needs only its own expanded channel, so the expanded channels are cut into ranges of whole
// 32-channel blocks as well: a workgroup is (tile, channel range), which keeps its LDS image small (four or more
// workgroups share a CU and overlap their stages) on layers with many channels; the input pixels are then staged once
// per range, which costs little (they are the narrow side of an expansion).
// Both stages produce bit for bit what the two stand-alone launches produce.
#include <type_traits>

#include "eh_internal.h"

namespace eh {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

namespace {

struct BlockGeom {
    int32_t th, tw;      // output rows and columns per workgroup
    int32_t tiles_y, tiles_w;  // workgroups per image, down and across
    int32_t ih, iwp;     // rows and columns of the expanded image a workgroup holds
    int32_t pixels;      // ih * iwp
    int32_t c;           // expanded channels of the layer
    int32_t nb;          // channel blocks of 32 per workgroup (grid y walks the ranges); bytes per pixel of the LDS image = 32 nb
    int32_t ks;          // reduction steps of 32 bytes of the pointwise stage
    int32_t cpitch;      // bytes per pixel of the LDS image
    int32_t tiles_x;     // depthwise tiles of four output columns per row of the workgroup's tile
    int32_t units_per_cq;  // th * tiles_x: depthwise thread-units per channel quad
    int32_t total_tiles; // n * tiles_y * tiles_w
    int32_t a_pitch;     // LDS bytes per input pixel: 32 ks + 16 (the slack spreads the fragment reads over the banks)
    FastDiv div_iwp, div_tx, div_tiles_y, div_tiles_w, div_ppp;
    FastDiv div_cq, div_cq_last;  // by the channel quads of a full range, and of the last one
    uint32_t a_off;      // byte offset of the staged input pixels
    uint32_t image_off;  // byte offset of the LDS image behind the staged weights, bias and input pixels
};

__device__ __forceinline__ int udot4(uint32_t a, uint32_t b, int acc) { return (int)__builtin_amdgcn_udot4(a, b, (uint32_t)acc, false); }

// the four channels of a column's three rows as four words of three bytes each (byte 3 zero)
__device__ __forceinline__ void column_words(uint32_t r0, uint32_t r1, uint32_t r2, uint32_t (&out)[4]) {
    const uint32_t t01 = __builtin_amdgcn_perm(r1, r0, 0x05010400u);
    const uint32_t t23 = __builtin_amdgcn_perm(r1, r0, 0x07030602u);
    out[0] = __builtin_amdgcn_perm(r2, t01, 0x0c040100u);
    out[1] = __builtin_amdgcn_perm(r2, t01, 0x0c050302u);
    out[2] = __builtin_amdgcn_perm(r2, t23, 0x0c060100u);
    out[3] = __builtin_amdgcn_perm(r2, t23, 0x0c070302u);
}

// S: depthwise stride.  FOLD: the depthwise stage multiplies raw bytes (unsigned form, weights of any range) instead of
// a - 128 against w - zp_w.  ROWSUM: the pointwise weights' zero point is not 128, so a pixel's byte sum enters.
// QM: pointwise requantization, 0 two-step order, 1 / 2 the single-shift forms.  KS: reduction steps of the pointwise
// stage when they are 1, 2 or 3 (a lane then keeps its pixel's operand bytes in registers across the channel blocks),
// 0 for any number (read from LDS for every product).
template <int S, bool FOLD, bool ROWSUM, int QM, int KS, bool PC>
__global__ __launch_bounds__(256) void pwdw_block_kernel(const GemmProblem pw, const DwProblem dw, const BlockGeom g) {
    const int ksteps = KS ? KS : g.ks;
    extern __shared__ __align__(16) uint8_t lds_raw[];
    v4i *b_s = reinterpret_cast<v4i *>(lds_raw);                              // [nb][ks][64 lanes]: pointwise weights, fragment order
    int32_t *bias_s = reinterpret_cast<int32_t *>(lds_raw + (size_t)g.nb * ksteps * 1024);  // [nb * 32]
    // PC (one multiplier and shift per channel in both operators): the pointwise stage's pairs beside the bias, as the
    // single-shift form's table (multiplier, right shift - 1, high word of the rounding term) or, two-step, as they are
    int32_t *pcm_s = bias_s + g.nb * 32, *pcf_s = pcm_s + g.nb * 32, *pch_s = pcf_s + g.nb * 32;
    uint8_t *img_s = lds_raw + g.image_off;                                   // [ih][iwp][cpitch] uint8 (xor 0x80 for the signed form)
    const int nb_first = blockIdx.y * g.nb;                                   // this workgroup's channel range
    const int c_first = nb_first * 32;
    const int c_here = g.c - c_first < g.nb * 32 ? g.c - c_first : g.nb * 32;  // channels of the range that exist (a multiple of 16)
    const int nb_here = (c_here + 31) >> 5;
    const int cpitch = g.cpitch;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, half = lane >> 5;
    // every XCD takes a contiguous eighth of the tiles: the rows two neighbouring tiles share are then fetched into one L2
    const uint32_t tile = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    if (tile >= (uint32_t)g.total_tiles) return;
    const uint32_t t_row = fastdiv(tile, g.div_tiles_w);
    const int txw = (int)(tile - t_row * (uint32_t)g.tiles_w);
    const uint32_t img = fastdiv(t_row, g.div_tiles_y);
    const int ty = (int)(t_row - img * (uint32_t)g.tiles_y);
    const int oy0 = ty * g.th, ox_first = txw * g.tw;
    const int iy_first = oy0 * S - dw.pad_t, ix_first = ox_first * S - dw.pad_l;  // image coordinates of the LDS image's corner
    uint8_t *a_s = lds_raw + g.a_off;  // [pixels][a_pitch]: the input pixels' reduction bytes as signed operands (a ^ 0x80), 0 past the reduction length

    // ---- stage 0: weights, bias and the tile's input pixels into LDS (8-byte pieces: pixels start on 8-byte boundaries)
    auto inside_image = [&](int q, int &iy, int &ix) {
        const int ry = (int)fastdiv((uint32_t)q, g.div_iwp), rx = q - ry * g.iwp;
        iy = iy_first + ry;
        ix = ix_first + rx;
        return (unsigned)iy < (unsigned)pw.h && (unsigned)ix < (unsigned)pw.w;
    };
    {
        const int ppp = ksteps * 4;  // 8-byte pieces per pixel
        const int pieces = g.pixels * ppp;
        for (int i = tid; i < pieces; i += 256) {
            const int q = KS ? i / (KS * 4) : (int)fastdiv((uint32_t)i, g.div_ppp), piece = i - q * ppp;
            int iy, ix;
            uint2 v = make_uint2(0u, 0u);  // bytes past the reduction length, and whole pixels outside the image: operand 0
            if (inside_image(q, iy, ix) && piece * 8 < pw.k) {
                v = *reinterpret_cast<const uint2 *>(pw.a + (((img * (uint32_t)pw.h + (uint32_t)iy) * (uint32_t)pw.w + (uint32_t)ix) * (uint32_t)pw.cin +
                                                               (uint32_t)pw.a_offset + (uint32_t)piece * 8u));
                v.x ^= pw.a_xor;
                v.y ^= pw.a_xor;
            }
            *reinterpret_cast<uint2 *>(a_s + q * g.a_pitch + piece * 8) = v;
        }
        const v4i *src = reinterpret_cast<const v4i *>(pw.b) + (size_t)nb_first * ksteps * 64;
        for (int i = tid; i < nb_here * ksteps * 64; i += 256) b_s[i] = src[i];
        for (int i = tid; i < nb_here * 32; i += 256) bias_s[i] = pw.bias[c_first + i];
        if constexpr (PC) {  // (the per-channel arrays are padded to whole channel blocks)
            for (int i = tid; i < nb_here * 32; i += 256) {
                const int32_t m = pw.rq.pc_multiplier[c_first + i], sh = pw.rq.pc_shift[c_first + i];
                pcm_s[i] = m;
                pcf_s[i] = QM != 0 ? -sh - 1 : sh;
                pch_s[i] = QM != 0 ? channel_table_pos_hi(pw.rq.zp_out, -sh) : 0;
            }
        }
        __syncthreads();
    }

    // ---- stage 1: the expanded pixels into the LDS image.  Units of (pixel block, channel block), a contiguous share per wave.
    const uint32_t flip_store = FOLD ? 0u : 0x80808080u;  // the signed depthwise form reads a - 128
    const uint32_t pad_word = ((uint32_t)dw.zp_in * 0x01010101u) ^ flip_store;
    const int blocks = (g.pixels + 31) >> 5;
    const RequantDev rq = pw.rq;
    {
        const int all = blocks * nb_here;
        const int first = (all * wave) >> 2, last = (all * (wave + 1)) >> 2;
        int blk = first / nb_here, nb = first - blk * nb_here;
        int loaded = -1, ncorr = 0, q = 0;
        bool ok = false;
        const uint8_t *arow = a_s;
        v4i held[KS ? KS : 1];
        for (int u = first; u < last; ++u) {
            if (blk != loaded) {  // this lane's pixel of the block: where its fragment bytes sit, its row-sum term, its place in the image
                loaded = blk;
                q = blk * 32 + r;
                int iy, ix;
                ok = q < g.pixels && inside_image(q, iy, ix);
                arow = a_s + (q < g.pixels ? q : g.pixels - 1) * g.a_pitch + half * 16;
                if constexpr (KS != 0) {
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) held[ks] = *reinterpret_cast<const v4i *>(arow + ks * 32);
                }
                if constexpr (ROWSUM) {
                    int rowsum = 0;
#pragma unroll
                    for (int ks = 0; ks < ksteps; ++ks) {
                        const v4i af = KS ? held[KS ? ks : 0] : *reinterpret_cast<const v4i *>(arow + ks * 32);
                        rowsum = __builtin_amdgcn_sdot4(af.x, 0x01010101, rowsum, false);
                        rowsum = __builtin_amdgcn_sdot4(af.y, 0x01010101, rowsum, false);
                        rowsum = __builtin_amdgcn_sdot4(af.z, 0x01010101, rowsum, false);
                        rowsum = __builtin_amdgcn_sdot4(af.w, 0x01010101, rowsum, false);
                    }
                    rowsum += __shfl_xor(rowsum, 32);  // the other half of every step's bytes
                    ncorr = -pw.zw * rowsum;
                }
            }
            const int32_t *bsrc = bias_s + nb * 32 + half * 16;
            v16i acc;
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
                const int4 bb = *reinterpret_cast<const int4 *>(bsrc + gq * 4);
                acc[gq * 4 + 0] = bb.x;
                acc[gq * 4 + 1] = bb.y;
                acc[gq * 4 + 2] = bb.z;
                acc[gq * 4 + 3] = bb.w;
            }
            const v4i *bw = b_s + nb * ksteps * 64 + lane;
            if constexpr (KS != 0) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(bw[ks * 64], held[ks], acc, 0, 0, 0);
            } else {
                for (int ks = 0; ks < ksteps; ++ks)
                    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(bw[ks * 64], *reinterpret_cast<const v4i *>(arow + ks * 32), acc, 0, 0, 0);
            }
            uint32_t packed[4];
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
                if constexpr (PC) {
                    const int tab = nb * 32 + half * 16 + gq * 4;
                    const int4 cm = *reinterpret_cast<const int4 *>(pcm_s + tab);
                    const int4 cf = *reinterpret_cast<const int4 *>(pcf_s + tab);
                    uint32_t o0, o1, o2, o3;
                    if constexpr (QM != 0) {
                        const int4 ch = *reinterpret_cast<const int4 *>(pch_s + tab);
                        o0 = requant_u8_channel_table<QM>(acc[gq * 4 + 0] + ncorr, cm.x, cf.x, ch.x, rq);
                        o1 = requant_u8_channel_table<QM>(acc[gq * 4 + 1] + ncorr, cm.y, cf.y, ch.y, rq);
                        o2 = requant_u8_channel_table<QM>(acc[gq * 4 + 2] + ncorr, cm.z, cf.z, ch.z, rq);
                        o3 = requant_u8_channel_table<QM>(acc[gq * 4 + 3] + ncorr, cm.w, cf.w, ch.w, rq);
                    } else {
                        o0 = requant_u8_channel(acc[gq * 4 + 0] + ncorr, cm.x, cf.x, rq);
                        o1 = requant_u8_channel(acc[gq * 4 + 1] + ncorr, cm.y, cf.y, rq);
                        o2 = requant_u8_channel(acc[gq * 4 + 2] + ncorr, cm.z, cf.z, rq);
                        o3 = requant_u8_channel(acc[gq * 4 + 3] + ncorr, cm.w, cf.w, rq);
                    }
                    packed[gq] = pack_bytes(o0, o1, o2, o3);
                } else if constexpr (QM != 0) {
                    packed[gq] = requant4_fast<QM>(acc[gq * 4 + 0], acc[gq * 4 + 1], acc[gq * 4 + 2], acc[gq * 4 + 3], ncorr, rq);
                } else {
                    packed[gq] = pack_bytes(requant_u8(acc[gq * 4 + 0] + ncorr, rq), requant_u8(acc[gq * 4 + 1] + ncorr, rq),
                                            requant_u8(acc[gq * 4 + 2] + ncorr, rq), requant_u8(acc[gq * 4 + 3] + ncorr, rq));
                }
            }
            if (q < g.pixels && nb * 32 + half * 16 < c_here) {  // (channel counts are multiples of 16: a lane's sixteen channels exist or do not)
                const uint4 v = ok ? make_uint4(packed[0] ^ flip_store, packed[1] ^ flip_store, packed[2] ^ flip_store, packed[3] ^ flip_store)
                                   : make_uint4(pad_word, pad_word, pad_word, pad_word);
                *reinterpret_cast<uint4 *>(img_s + (uint32_t)q * (uint32_t)cpitch + (uint32_t)(nb * 32 + half * 16)) = v;
            }
            if (++nb == nb_here) {
                nb = 0;
                ++blk;
            }
        }
    }
    __syncthreads();

    // ---- stage 2: the depthwise outputs from the LDS image
    constexpr int TW = 4, IW = (TW - 1) * S + 3;  // a thread's four adjacent output pixels
    const uint32_t cq_count = (uint32_t)c_here >> 2;
    const uint32_t units = (uint32_t)g.units_per_cq * cq_count;
    const uint32_t cq_first = (uint32_t)c_first >> 2;
    const RequantDev drq = dw.rq;
    const FastDiv div_cq = blockIdx.y + 1 == gridDim.y ? g.div_cq_last : g.div_cq;
    for (uint32_t u = (uint32_t)tid; u < units; u += 256u) {
        const uint32_t t = fastdiv(u, div_cq);
        const uint32_t cql = u - t * cq_count, cq = cq_first + cql;  // channel quad within the range, and in the layer
        const uint32_t row = fastdiv(t, g.div_tx);
        const int tx = (int)(t - row * (uint32_t)g.tiles_x);
        const int oy = oy0 + (int)row, lx0 = tx * TW, ox0 = ox_first + lx0;  // lx0: first column within the workgroup's tile
        if (oy >= dw.ho) continue;
        uint32_t in[3][IW];
#pragma unroll
        for (int ky = 0; ky < 3; ++ky)
#pragma unroll
            for (int x = 0; x < IW; ++x) {
                int col = lx0 * S + x;
                col = col < g.iwp ? col : g.iwp - 1;  // columns past the last window belong to outputs that are not stored
                in[ky][x] = *reinterpret_cast<const uint32_t *>(img_s + (((int)row * S + ky) * g.iwp + col) * cpitch + (int)cql * 4);
            }
        int4 wk[3];
#pragma unroll
        for (int kx = 0; kx < 3; ++kx) wk[kx] = *reinterpret_cast<const int4 *>((FOLD ? dw.w_fold : dw.w_trip) + ((uint32_t)kx * (uint32_t)dw.cout + cq * 4u));
        const int4 b4 = *reinterpret_cast<const int4 *>((FOLD ? dw.bias_fold : dw.bias_trip) + cq * 4u);
        int4 dm = make_int4(0, 0, 0, 0), ds = dm;  // PC: the depthwise stage's four pairs
        if constexpr (PC) {
            dm = *reinterpret_cast<const int4 *>(drq.pc_multiplier + cq * 4u);
            ds = *reinterpret_cast<const int4 *>(drq.pc_shift + cq * 4u);
        }
        uint32_t colw[IW][4];
        int cs[FOLD ? IW : 1][4];
#pragma unroll
        for (int x = 0; x < IW; ++x) {
            column_words(in[0][x], in[1][x], in[2][x], colw[x]);
            if constexpr (FOLD) {
#pragma unroll
                for (int c = 0; c < 4; ++c) cs[x][c] = udot4(colw[x][c], 0x00010101u, 0);
            }
        }
        uint8_t *dst = dw.out + (((img * (uint32_t)dw.ho + (uint32_t)oy) * (uint32_t)dw.wo + (uint32_t)ox0) * (uint32_t)dw.cout + cq * 4u);
#pragma unroll
        for (int j = 0; j < TW; ++j) {
            int acc0 = b4.x, acc1 = b4.y, acc2 = b4.z, acc3 = b4.w;
#pragma unroll
            for (int kx = 0; kx < 3; ++kx) {
                if constexpr (FOLD) {
                    acc0 = udot4(colw[j * S + kx][0], (uint32_t)wk[kx].x, acc0);
                    acc1 = udot4(colw[j * S + kx][1], (uint32_t)wk[kx].y, acc1);
                    acc2 = udot4(colw[j * S + kx][2], (uint32_t)wk[kx].z, acc2);
                    acc3 = udot4(colw[j * S + kx][3], (uint32_t)wk[kx].w, acc3);
                } else {
                    acc0 = __builtin_amdgcn_sdot4((int)colw[j * S + kx][0], wk[kx].x, acc0, false);
                    acc1 = __builtin_amdgcn_sdot4((int)colw[j * S + kx][1], wk[kx].y, acc1, false);
                    acc2 = __builtin_amdgcn_sdot4((int)colw[j * S + kx][2], wk[kx].z, acc2, false);
                    acc3 = __builtin_amdgcn_sdot4((int)colw[j * S + kx][3], wk[kx].w, acc3, false);
                }
            }
            if constexpr (FOLD) {
                acc0 += __mul24(-dw.zp_w, cs[j * S][0] + cs[j * S + 1][0] + cs[j * S + 2][0]);
                acc1 += __mul24(-dw.zp_w, cs[j * S][1] + cs[j * S + 1][1] + cs[j * S + 2][1]);
                acc2 += __mul24(-dw.zp_w, cs[j * S][2] + cs[j * S + 1][2] + cs[j * S + 2][2]);
                acc3 += __mul24(-dw.zp_w, cs[j * S][3] + cs[j * S + 1][3] + cs[j * S + 2][3]);
            }
            uint32_t o;
            if constexpr (PC) {
                if (drq.fast == 2)
                    o = pack_bytes(requant_u8_channel_fast<2>(acc0, dm.x, ds.x, drq), requant_u8_channel_fast<2>(acc1, dm.y, ds.y, drq),
                                   requant_u8_channel_fast<2>(acc2, dm.z, ds.z, drq), requant_u8_channel_fast<2>(acc3, dm.w, ds.w, drq));
                else if (drq.fast)
                    o = pack_bytes(requant_u8_channel_fast<1>(acc0, dm.x, ds.x, drq), requant_u8_channel_fast<1>(acc1, dm.y, ds.y, drq),
                                   requant_u8_channel_fast<1>(acc2, dm.z, ds.z, drq), requant_u8_channel_fast<1>(acc3, dm.w, ds.w, drq));
                else
                    o = pack_bytes(requant_u8_channel(acc0, dm.x, ds.x, drq), requant_u8_channel(acc1, dm.y, ds.y, drq),
                                   requant_u8_channel(acc2, dm.z, ds.z, drq), requant_u8_channel(acc3, dm.w, ds.w, drq));
            } else if (drq.fast == 2)
                o = requant4_fast<2>(acc0, acc1, acc2, acc3, 0, drq);
            else if (drq.fast)
                o = requant4_fast<1>(acc0, acc1, acc2, acc3, 0, drq);
            else
                o = pack_bytes(requant_u8(acc0, drq), requant_u8(acc1, drq), requant_u8(acc2, drq), requant_u8(acc3, drq));
            if (lx0 + j < g.tw && ox0 + j < dw.wo) *reinterpret_cast<uint32_t *>(dst + (uint32_t)j * (uint32_t)dw.cout) = o;
        }
    }
}

constexpr size_t kBlockLdsMax = 150 * 1024;

// Bytes per pixel of the LDS image for `nb` channel blocks of a layer of c channels: the channels of the widest range,
// stretched where needed so that the pitch in words is an odd multiple of four (stage 1 writes sixteen bytes per lane
// for 32 consecutive pixels; at an even multiple of four words those writes meet in a quarter of the banks).
int block_image_pitch(int nb, int c) {
    int words = (nb * 32 < c ? nb * 32 : c) / 4;
    if ((words & 7) == 0) words += 4;
    return words * 4;
}

size_t block_lds_bytes(int nb, int ks, int ih, int iwp, int c, uint32_t *a_off, uint32_t *image_off) {
    const size_t head = ((size_t)nb * ks * 1024 + (size_t)nb * 512 + 15) & ~(size_t)15;  // weights, bias, three per-channel tables
    const size_t a_bytes = ((size_t)ih * iwp * (ks * 32 + 16) + 15) & ~(size_t)15;
    if (a_off) *a_off = (uint32_t)head;
    if (image_off) *image_off = (uint32_t)(head + a_bytes);
    return head + a_bytes + (size_t)ih * iwp * block_image_pitch(nb, c);
}

}  // namespace

// The pointwise problem is a one-tap problem of at most eight 32-byte reduction steps on whole dense images whose
// weights are packed in fragment order, the depthwise one a 3x3 channels-last layer of stride 1 or 2 on the pointwise
// output with the 8-bit dot product weights at hand; uint8 tensors; one requantization pair per operator, or one pair per
// channel in both.
bool pwdw_block_applies(const GemmProblem &pw, const DwProblem &dw) {
    if (pw.cfg.id != GEMM_THIN || pw.k_pad > 256 || pw.k > pw.k_pad || (pw.k & 7) != 0 || (pw.cin & 7) != 0 || pw.k != pw.cin) return false;
    if (pw.stride_h != 1 || pw.stride_w != 1 || pw.y_base != 0 || pw.x_base != 0 || pw.ho != pw.h || pw.wo != pw.w) return false;
    if (pw.a_xor != 0x80808080u || pw.out_xor != 0u || pw.residual) return false;
    if ((pw.rq.pc_multiplier != nullptr) != (dw.rq.pc_multiplier != nullptr)) return false;
    if (dw.kh != 3 || dw.kw != 3 || dw.dil_h != 1 || dw.dil_w != 1 || dw.stride_h != dw.stride_w || (dw.stride_h != 1 && dw.stride_h != 2)) return false;
    if (dw.dm != 1 || dw.c != dw.cout || dw.c != pw.n || (dw.c & 15) != 0 || dw.h != pw.h || dw.w_ != pw.w) return false;
    if (dw.io_flip || (!dw.w_trip && !dw.w_fold)) return false;
    if (dw.pad_t < 0 || dw.pad_l < 0 || dw.pad_t > 2 || dw.pad_l > 2) return false;
    if ((size_t)dw.n * dw.h * dw.w_ * pw.cin >= (1ull << 31) || (size_t)dw.n * dw.ho * dw.wo * dw.cout >= (1ull << 31)) return false;
    return block_lds_bytes(1, pw.k_pad / 32, 3, 3 * dw.stride_w + 3, dw.c, nullptr, nullptr) <= kBlockLdsMax;  // one row of four outputs, one channel block
}

// Whether the one launch beats the two.  The fused kernel computes the expanded pixels of a tile's halo twice and
// requantizes every expanded value on the vector ALU just as the stand-alone kernels do, so what it saves is the
// expanded tensor's trip through memory and one launch; whether that pays depends on the shape, and the answer here
// is a table of the shapes that were timed inside a network (MobileNetV2 at 224 x 224, 32 images per launch, each
// pair switched to the fused kernel on its own; microseconds per network pass against 445):
//   image  in -> expanded  stride   change        image  in -> expanded  stride   change
//   112     16 ->  96        2      +1.9           14    64 -> 384         1      -6.1 / -5.0 / -5.4 / -3.8
//    56     24 -> 144        1      -0.8           14    96 -> 576         1      +0.1 / -0.4
//    56     24 -> 144        2      -6.9           14    96 -> 576         2      -1.5
//    28     32 -> 192        1      -5.2 / -3.8     7   160 -> 960         1      +0.4 / -0.6 / -0.4
//    28     32 -> 192        2      -6.4
// (changes within +-1.5 are noise; the listed shapes are the ones beyond it.)
// A shape that is not in the table runs as two launches.
bool pwdw_block_listed(int32_t images, int32_t image_h, int32_t image_w, int32_t in_channels, int32_t expanded_channels, int32_t stride) {
    // Below 32 images a launch is mostly latency, and one launch instead of two wins for every pair the kernel fits:
    // MobileNetV2 with all 16 fitting pairs fused against the listed ones, 198 against 220 us at batch 1, 209 against 256
    // at 4, 247 against 263 at 8, 287 against 294 at 16, 325 against 328 at 24; at 32 the list wins, 350 against 354.
    if (images < 32) return true;
    if (image_h != image_w) return false;
    struct Shape {
        int32_t image, in, expanded, stride;
    };
    static const Shape faster[] = {{56, 24, 144, 2}, {28, 32, 192, 1}, {28, 32, 192, 2}, {14, 64, 384, 1}};
    for (const Shape &s : faster)
        if (image_h == s.image && in_channels == s.in && expanded_channels == s.expanded && stride == s.stride) return true;
    return false;
}

bool pwdw_block_preferred(const GemmProblem &pw, const DwProblem &dw) {
    return pwdw_block_applies(pw, dw) && pwdw_block_listed(dw.n, dw.h, dw.w_, pw.k, dw.c, dw.stride_h);
}

// rows_per_tile / cols_per_tile: the tile a workgroup owns, 0 = chosen here
int launch_pwdw_block(const GemmProblem &pw, const DwProblem &caller_dw, int rows_per_tile, int cols_per_tile, hipStream_t stream) {
    EH_REQUIRE(pwdw_block_applies(pw, caller_dw), "block: the two operators do not fit the fused kernel");
    EH_REQUIRE((reinterpret_cast<uintptr_t>(pw.a) & 7) == 0 && (reinterpret_cast<uintptr_t>(caller_dw.out) & 3) == 0, "block: unaligned tensors");
    DwProblem dw = caller_dw;
    if (dw.w_trip) dw.w_fold = nullptr;                 // the signed form where it applies, as the stand-alone launcher decides
    if (dw.w_fold) dw.zp_w += dw.w_signed ? 128 : 0;    // zero point of the uint8 values the unsigned form multiplies
    const int S = dw.stride_h;
    BlockGeom g;
    g.c = dw.c;
    g.ks = pw.k_pad / 32;
    g.a_pitch = g.ks * 32 + 16;
    const int nb_all = (dw.c + 31) / 32;
    // Tile shape and channel blocks per workgroup.  A workgroup's three stages run one after the other, so the stages
    // of different workgroups have to overlap on a CU: the shapes considered leave room for four or more workgroups in
    // a CU's LDS (measured: tiles of twice that size take twice as long at a batch of 256, however little halo they
    // recompute) and, where the problem is large enough, give the launch at least three workgroups per CU.  Among those
    // the one that computes the fewest pixel slots wins, counting the slots that pixel blocks of 32 and output tiles of
    // four leave empty and, at a lower weight, the input bytes staged again for every channel range.
    int th = rows_per_tile, tw = cols_per_tile, nb = nb_all;
    {
        double best = -1;
        int best_th = 1, best_tw = dw.wo < 4 ? dw.wo : 4, best_nb = 1;
        for (int pass = 0; pass < 3 && best < 0; ++pass)  // later passes: fewer workgroups, then anything that fits at all
            for (int cn = 1; cn <= nb_all; ++cn) {
                const int ranges = (nb_all + cn - 1) / cn;
                if ((ranges - 1) * cn >= nb_all) continue;  // the same ranges with fewer blocks each
                for (int ch = 1; ch <= dw.ho && ch <= 16; ++ch)
                    for (int cw = 1; cw <= dw.wo && cw <= 64; ++cw) {
                        if (rows_per_tile > 0 && ch != rows_per_tile) continue;
                        if (cols_per_tile > 0 && cw != cols_per_tile) continue;
                        const int ih = (ch - 1) * S + 3, iw = (cw - 1) * S + 3;
                        const size_t lds = block_lds_bytes(cn, g.ks, ih, iw, dw.c, nullptr, nullptr);
                        if (pass < 2 ? lds * 4 > 144 * 1024 : lds > kBlockLdsMax) continue;
                        const long wgs = (long)dw.n * ((dw.ho + ch - 1) / ch) * ((dw.wo + cw - 1) / cw) * ranges;
                        if (pass == 0 && wgs < 768) continue;
                        const int px = ih * iw;
                        const double tiles = (double)dw.n * ((dw.ho + ch - 1) / ch) * ((dw.wo + cw - 1) / cw);
                        const double stage1 = (double)((px + 31) / 32 * 32) * tiles / ((double)dw.n * dw.h * dw.w_);   // pixel slots computed per real pixel
                        const double stage2 = (double)ch * ((cw + 3) / 4 * 4) * tiles / ((double)dw.n * dw.ho * dw.wo);  // output slots per real output
                        const double restage = (double)px * tiles * ranges * (g.ks * 32) / ((double)dw.n * dw.h * dw.w_ * dw.c);  // staged input bytes per expanded byte
                        const double cost = stage1 + 0.5 * stage2 + 2.0 * restage;
                        if (best < 0 || cost < best) {
                            best = cost;
                            best_th = ch;
                            best_tw = cw;
                            best_nb = cn;
                        }
                    }
            }
        EH_REQUIRE(best >= 0, "block: no tile of the requested shape fits LDS");
        th = best_th;
        tw = best_tw;
        nb = best_nb;
    }
    g.nb = nb;
    EH_REQUIRE(th >= 1 && th <= dw.ho && tw >= 1 && tw <= dw.wo, "block: tile of %d x %d outputs", th, tw);
    g.th = th;
    g.tw = tw;
    g.ih = (th - 1) * S + 3;
    g.iwp = (tw - 1) * S + 3;
    g.pixels = g.ih * g.iwp;
    g.tiles_x = (tw + 3) / 4;
    g.tiles_y = (dw.ho + th - 1) / th;
    g.tiles_w = (dw.wo + tw - 1) / tw;
    g.total_tiles = dw.n * g.tiles_y * g.tiles_w;
    g.units_per_cq = th * g.tiles_x;
    g.div_iwp = make_fastdiv((uint32_t)g.iwp);
    g.div_tx = make_fastdiv((uint32_t)g.tiles_x);
    g.div_tiles_y = make_fastdiv((uint32_t)g.tiles_y);
    g.div_tiles_w = make_fastdiv((uint32_t)g.tiles_w);
    g.div_ppp = make_fastdiv((uint32_t)(g.ks * 4));
    const int ranges = (nb_all + g.nb - 1) / g.nb;
    g.div_cq = make_fastdiv((uint32_t)(g.nb * 8 < g.c / 4 ? g.nb * 8 : g.c / 4));
    g.div_cq_last = make_fastdiv((uint32_t)((g.c - (ranges - 1) * g.nb * 32) / 4));
    g.cpitch = block_image_pitch(g.nb, g.c);
    const size_t lds = block_lds_bytes(g.nb, g.ks, g.ih, g.iwp, g.c, &g.a_off, &g.image_off);
    EH_REQUIRE(lds <= kBlockLdsMax, "block: %zu bytes of LDS", lds);
    if (g.total_tiles <= 0) return EH_OK;
    const dim3 grid((unsigned)((g.total_tiles + 7) / 8 * 8), (unsigned)ranges);
    auto launch_pc = [&](auto s_c, auto fold_c, auto rowsum_c, auto qm_c, auto ks_c, auto pc_c) {
        auto kernel = pwdw_block_kernel<decltype(s_c)::value, decltype(fold_c)::value, decltype(rowsum_c)::value, decltype(qm_c)::value, decltype(ks_c)::value,
                                        decltype(pc_c)::value>;
        if (lds > 64 * 1024) {
            // (a driver call, made per launch of the tall-tile shapes only; the default tile height stays below 64 KiB)
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kBlockLdsMax);
            if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(pwdw_block_kernel)");
        }
        hipLaunchKernelGGL(kernel, grid, dim3(256), lds, stream, pw, dw, g);
        return (int)EH_OK;
    };
    auto launch = [&](auto s_c, auto fold_c, auto rowsum_c, auto qm_c, auto ks_c) {
        return pw.rq.pc_multiplier ? launch_pc(s_c, fold_c, rowsum_c, qm_c, ks_c, std::true_type{}) : launch_pc(s_c, fold_c, rowsum_c, qm_c, ks_c, std::false_type{});
    };
    auto with_ks = [&](auto s_c, auto fold_c, auto rowsum_c, auto qm_c) {
        if (g.ks == 1) return launch(s_c, fold_c, rowsum_c, qm_c, std::integral_constant<int, 1>{});
        if (g.ks == 2) return launch(s_c, fold_c, rowsum_c, qm_c, std::integral_constant<int, 2>{});
        if (g.ks == 3) return launch(s_c, fold_c, rowsum_c, qm_c, std::integral_constant<int, 3>{});
        return launch(s_c, fold_c, rowsum_c, qm_c, std::integral_constant<int, 0>{});
    };
    auto with_qm = [&](auto s_c, auto fold_c, auto rowsum_c) {
        if (pw.rq.fast == 2) return with_ks(s_c, fold_c, rowsum_c, std::integral_constant<int, 2>{});
        if (pw.rq.fast == 1) return with_ks(s_c, fold_c, rowsum_c, std::integral_constant<int, 1>{});
        return with_ks(s_c, fold_c, rowsum_c, std::integral_constant<int, 0>{});
    };
    auto with_rowsum = [&](auto s_c, auto fold_c) {
        return pw.zw != 0 ? with_qm(s_c, fold_c, std::true_type{}) : with_qm(s_c, fold_c, std::false_type{});
    };
    auto with_fold = [&](auto s_c) { return dw.w_trip ? with_rowsum(s_c, std::false_type{}) : with_rowsum(s_c, std::true_type{}); };
    const int rc = S == 1 ? with_fold(std::integral_constant<int, 1>{}) : with_fold(std::integral_constant<int, 2>{});
    if (rc) return rc;
    EH_HIP(hipGetLastError());
    return EH_OK;
}

}  // namespace eh
