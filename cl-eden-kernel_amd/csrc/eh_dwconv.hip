// Depthwise uint8 convolution (gfx950): bandwidth-bound, no matrix cores.
//
// Replaces the reference's depthwise kernels for the uint8 path
// (gpu/operators/cl_kernels/DepthwiseconvolutionKernels.cpp:1242-2290: generic
// depthwise_conv plus the 3x3 pad-merge specialisations) and their pad pass
// (PadConvertKernels.cpp:7-23).  Out-of-image taps read the input zero point,
// as the reference's padding does, so they contribute nothing.
//
// Channels-last fast path: one thread owns four adjacent channels of one output
// pixel, so a wavefront reads whole contiguous pixel rows.  Two taps of one
// channel are paired into a 16-bit dot product (v_dot2_i32_i16) against
// weights stored as (w - zp_w) int16 pairs; the input zero point is folded
// into the bias: sum (a - zi)(w - zw) = sum a (w - zw) - zi * sum (w - zw).
#include <type_traits>

#include "eh_internal.h"

namespace eh {
namespace {

typedef short v2s __attribute__((ext_vector_type(2)));

__device__ __forceinline__ int dot2(uint32_t a_pair, int32_t w_pair, int acc) {
    return __builtin_amdgcn_sdot2(__builtin_bit_cast(v2s, a_pair), __builtin_bit_cast(v2s, w_pair), acc, false);
}

// byte j of `lo` into bits 0..15 and byte j of `hi` into bits 16..31, zero extended
template <int J>
__device__ __forceinline__ uint32_t pair_bytes(uint32_t lo, uint32_t hi) {
    constexpr uint32_t sel = (0x0cu << 24) | ((4u + J) << 16) | (0x0cu << 8) | (uint32_t)J;
    return __builtin_amdgcn_perm(hi, lo, sel);
}

// The per-channel multipliers and shifts of four adjacent channels, read once per thread.
struct ChannelQuad {
    int4 m, s;
};
template <bool PC>
__device__ __forceinline__ ChannelQuad load_channel_quad(const RequantDev &rq, uint32_t ch) {
    ChannelQuad q{};
    if (PC && rq.pc_multiplier) {
        q.m = *reinterpret_cast<const int4 *>(rq.pc_multiplier + ch);
        q.s = *reinterpret_cast<const int4 *>(rq.pc_shift + ch);
    }
    return q;
}

// Four adjacent channels' accumulators to four output bytes.  With one multiplier and shift per channel
// (depthwise_conv_per_channel, gpu/operators/cl_kernels/DepthwiseconvolutionKernels.cpp:1323-1371) the four pairs
// come in `cq`.
template <bool PC = true>
__device__ __forceinline__ uint32_t requant4(int acc0, int acc1, int acc2, int acc3, const RequantDev &rq, const ChannelQuad &cq) {
    if (PC && rq.pc_multiplier)  // the two-step order; the single-shift form per channel is the dot product kernel's
        return pack_bytes(requant_u8_channel(acc0, cq.m.x, cq.s.x, rq), requant_u8_channel(acc1, cq.m.y, cq.s.y, rq),
                          requant_u8_channel(acc2, cq.m.z, cq.s.z, rq), requant_u8_channel(acc3, cq.m.w, cq.s.w, rq));
    if (rq.fast == 2) return requant4_fast<2>(acc0, acc1, acc2, acc3, 0, rq);
    if (rq.fast) return requant4_fast<1>(acc0, acc1, acc2, acc3, 0, rq);
    return pack_bytes(requant_u8(acc0, rq), requant_u8(acc1, rq), requant_u8(acc2, rq), requant_u8(acc3, rq));
}

// the per-channel single-shift form alone (rq.fast is 1 or 2)
__device__ __forceinline__ uint32_t requant4_channel_fast(int acc0, int acc1, int acc2, int acc3, const RequantDev &rq, const ChannelQuad &cq) {
    if (rq.fast == 2)
        return pack_bytes(requant_u8_channel_fast<2>(acc0, cq.m.x, cq.s.x, rq), requant_u8_channel_fast<2>(acc1, cq.m.y, cq.s.y, rq),
                          requant_u8_channel_fast<2>(acc2, cq.m.z, cq.s.z, rq), requant_u8_channel_fast<2>(acc3, cq.m.w, cq.s.w, rq));
    return pack_bytes(requant_u8_channel_fast<1>(acc0, cq.m.x, cq.s.x, rq), requant_u8_channel_fast<1>(acc1, cq.m.y, cq.s.y, rq),
                      requant_u8_channel_fast<1>(acc2, cq.m.z, cq.s.z, rq), requant_u8_channel_fast<1>(acc3, cq.m.w, cq.s.w, rq));
}

// Workgroups are dispatched round-robin over the 8 XCDs, each with its own L2.  Neighbouring output rows read
// the same input rows, so every XCD takes one contiguous eighth of the block range (launch grids are whole
// multiples of 8): a shared input row is then fetched from HBM into one L2 instead of two or three.
__device__ __forceinline__ uint32_t xcd_contiguous_block() { return (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3); }

// One output pixel's four adjacent channels per thread, any kernel size, stride and dilation (KH = 0: sizes from the
// problem).  SMALL: both tensors below 2^31 bytes, so the index is decoded with 32-bit multiplications and the taps'
// offsets are 32-bit (64-bit divisions and multiply-adds cost several times the rest of a small kernel's arithmetic).
template <int KH, int KW, bool SMALL>
__global__ __launch_bounds__(256) void dw_nhwc_vec4_kernel(const DwProblem p, const long total, const FastDiv div_cq, const FastDiv div_wo,
                                                           const FastDiv div_ho) {
    using Offset = std::conditional_t<SMALL, uint32_t, size_t>;
    const long idx = (long)xcd_contiguous_block() * 256 + threadIdx.x;
    if (idx >= total) return;
    const int cq_count = p.c >> 2;
    int cq, ox, oy, img;
    Offset pix;
    if constexpr (SMALL) {
        const uint32_t i = (uint32_t)idx, px = fastdiv(i, div_cq), t0 = fastdiv(px, div_wo), im = fastdiv(t0, div_ho);
        cq = (int)(i - px * (uint32_t)cq_count);
        ox = (int)(px - t0 * (uint32_t)p.wo);
        oy = (int)(t0 - im * (uint32_t)p.ho);
        img = (int)im;
        pix = px;
    } else {
        cq = (int)(idx % cq_count);
        const long px = idx / cq_count;
        ox = (int)(px % p.wo);
        const long t0 = px / p.wo;
        oy = (int)(t0 % p.ho), img = (int)(t0 / p.ho);
        pix = (Offset)px;
    }
    const int kh = KH ? KH : p.kh, kw = KW ? KW : p.kw;
    const int taps = kh * kw, pairs = (taps + 1) >> 1;
    const int iy0 = oy * p.stride_h - p.pad_t, ix0 = ox * p.stride_w - p.pad_l;
    const uint8_t *src = p.in + ((Offset)img * (Offset)(p.h * p.w_) * (Offset)p.c + (Offset)(cq * 4));
    const uint32_t fill = (uint32_t)p.zp_in * 0x01010101u;

    auto tap_at = [&](int ky, int kx) -> uint32_t {
        // loaded from a clamped address whatever the tap, so that the loads of several taps can be in flight together
        const int iy = iy0 + ky * p.dil_h, ix = ix0 + kx * p.dil_w;
        const int iyc = iy < 0 ? 0 : (iy >= p.h ? p.h - 1 : iy), ixc = ix < 0 ? 0 : (ix >= p.w_ ? p.w_ - 1 : ix);
        const uint32_t v = *reinterpret_cast<const uint32_t *>(src + ((Offset)iyc * (Offset)p.w_ + (Offset)ixc) * (Offset)p.c) ^ p.io_flip;
        return (unsigned)iy < (unsigned)p.h && (unsigned)ix < (unsigned)p.w_ ? v : fill;
    };
    const int4 b4 = *reinterpret_cast<const int4 *>(p.bias_folded + cq * 4);
    int acc0 = b4.x, acc1 = b4.y, acc2 = b4.z, acc3 = b4.w;
    auto accumulate = [&](int pr, uint32_t lo, uint32_t hi) {
        const int4 w4 = *reinterpret_cast<const int4 *>(p.w_pair + ((Offset)pr * (Offset)p.cout + (Offset)(cq * 4)));
        acc0 = dot2(pair_bytes<0>(lo, hi), w4.x, acc0);
        acc1 = dot2(pair_bytes<1>(lo, hi), w4.y, acc1);
        acc2 = dot2(pair_bytes<2>(lo, hi), w4.z, acc2);
        acc3 = dot2(pair_bytes<3>(lo, hi), w4.w, acc3);
    };
    if constexpr (KH != 0) {
#pragma unroll
        for (int pr = 0; pr < (KH * KW + 1) / 2; ++pr) {
            constexpr int kw_c = KW ? KW : 1;
            const int t = 2 * pr;
            accumulate(pr, tap_at(t / kw_c, t % kw_c), t + 1 < KH * KW ? tap_at((t + 1) / kw_c, (t + 1) % kw_c) : 0u);
        }
    } else {
        // taps in row-major order, two per step; (ky, kx) walk along without a division per tap
        int ky = 0, kx = 0;
        auto next = [&]() -> uint32_t {
            const uint32_t v = ky < kh ? tap_at(ky, kx) : 0u;
            if (++kx == kw) kx = 0, ++ky;
            return v;
        };
        int pr = 0;
        for (; pr + 4 <= pairs; pr += 4) {  // eight taps requested before the first is used
            uint32_t v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = next();
#pragma unroll
            for (int i = 0; i < 4; ++i) accumulate(pr + i, v[2 * i], v[2 * i + 1]);
        }
        for (; pr < pairs; ++pr) {
            const uint32_t lo = next(), hi = next();
            accumulate(pr, lo, hi);
        }
    }
    *reinterpret_cast<uint32_t *>(p.out + (pix * (Offset)p.cout + (Offset)(cq * 4))) =
        requant4(acc0, acc1, acc2, acc3, p.rq, load_channel_quad<true>(p.rq, (uint32_t)cq * 4u)) ^ p.io_flip;
}

// 3x3, dilation 1, stride S in both directions: a thread owns four adjacent channels of FOUR
// horizontally adjacent output pixels.  The 3 x (3 * S + 3) input pixels they need are loaded
// once (every load is issued before the first use, from clamped in-image addresses; taps
// outside the image are then replaced by the input zero point), so the address arithmetic, the
// weight and bias loads and the border tests are shared by sixteen outputs.
template <int S, bool PC, bool FLIP>
__global__ __launch_bounds__(256) void dw3x3_nhwc_tile4_kernel(const DwProblem p, const uint32_t total, const int tiles_x,
                                                               const FastDiv div_cq, const FastDiv div_tiles, const FastDiv div_ho) {
    constexpr int TW = 4, IW = (TW - 1) * S + 3;
    const uint32_t idx = xcd_contiguous_block() * 256u + threadIdx.x;
    if (idx >= total) return;
    // idx -> (image, output row, tile of four output columns, channel quad), channel quad fastest;
    // all offsets fit 32 bits (the launcher checks the tensor sizes)
    const uint32_t cq_count = (uint32_t)p.c >> 2;
    uint32_t r = fastdiv(idx, div_cq);
    const uint32_t cq = idx - r * cq_count;
    const uint32_t r2 = fastdiv(r, div_tiles);
    const int tx = (int)(r - r2 * (uint32_t)tiles_x);
    const uint32_t img = fastdiv(r2, div_ho);
    const int oy = (int)(r2 - img * (uint32_t)p.ho);
    const int ox0 = tx * TW;
    const int iy0 = oy * S - p.pad_t, ix0 = ox0 * S - p.pad_l;
    const uint32_t fill = (uint32_t)p.zp_in * 0x01010101u;
    const uint32_t base = img * (uint32_t)(p.h * p.w_ * p.c) + cq * 4u;

    uint32_t col_off[IW];
    bool col_ok[IW];
#pragma unroll
    for (int x = 0; x < IW; ++x) {
        const int ix = ix0 + x;
        col_ok[x] = (unsigned)ix < (unsigned)p.w_;
        const int ixc = ix < 0 ? 0 : (ix >= p.w_ ? p.w_ - 1 : ix);
        col_off[x] = base + (uint32_t)ixc * (uint32_t)p.c;
    }
    uint32_t in[3][IW];
#pragma unroll
    for (int ky = 0; ky < 3; ++ky) {
        const int iy = iy0 + ky;
        const bool row_ok = (unsigned)iy < (unsigned)p.h;
        const int iyc = iy < 0 ? 0 : (iy >= p.h ? p.h - 1 : iy);
        const uint32_t row_off = (uint32_t)iyc * (uint32_t)(p.w_ * p.c);
#pragma unroll
        for (int x = 0; x < IW; ++x) {
            const uint32_t v = *reinterpret_cast<const uint32_t *>(p.in + (row_off + col_off[x]));
            in[ky][x] = row_ok && col_ok[x] ? (FLIP ? v ^ 0x80808080u : v) : fill;
        }
    }
    int4 w4[5];
#pragma unroll
    for (int pr = 0; pr < 5; ++pr) w4[pr] = *reinterpret_cast<const int4 *>(p.w_pair + ((uint32_t)pr * (uint32_t)p.cout + cq * 4u));
    const int4 b4 = *reinterpret_cast<const int4 *>(p.bias_folded + cq * 4u);
    uint8_t *dst = p.out + (((img * (uint32_t)p.ho + (uint32_t)oy) * (uint32_t)p.wo + (uint32_t)ox0) * (uint32_t)p.cout + cq * 4u);
    const RequantDev rq = p.rq;
#pragma unroll
    for (int j = 0; j < TW; ++j) {
        int acc0 = b4.x, acc1 = b4.y, acc2 = b4.z, acc3 = b4.w;
#pragma unroll
        for (int pr = 0; pr < 5; ++pr) {
            const int t0 = 2 * pr, t1 = 2 * pr + 1;
            const uint32_t lo = in[t0 / 3][j * S + t0 % 3];
            const uint32_t hi = t1 < 9 ? in[t1 / 3][j * S + t1 % 3] : 0u;
            acc0 = dot2(pair_bytes<0>(lo, hi), w4[pr].x, acc0);
            acc1 = dot2(pair_bytes<1>(lo, hi), w4[pr].y, acc1);
            acc2 = dot2(pair_bytes<2>(lo, hi), w4[pr].z, acc2);
            acc3 = dot2(pair_bytes<3>(lo, hi), w4[pr].w, acc3);
        }
        uint32_t o = requant4<PC>(acc0, acc1, acc2, acc3, rq, load_channel_quad<PC>(rq, cq * 4u));
        if (FLIP) o ^= 0x80808080u;
        if (ox0 + j < p.wo) *reinterpret_cast<uint32_t *>(dst + (uint32_t)j * (uint32_t)p.cout) = o;
    }
}

// byte J of three rows' words into bytes 0, 1, 2 of one word (byte 3 zero): the three vertical taps of one channel
template <int J>
__device__ __forceinline__ uint32_t column_bytes(uint32_t r0, uint32_t r1, uint32_t r2) {
    constexpr uint32_t sel01 = (0x0cu << 24) | (0x0cu << 16) | ((4u + J) << 8) | (uint32_t)J;
    constexpr uint32_t sel2 = (0x0cu << 24) | ((4u + J) << 16) | (1u << 8) | 0u;
    return __builtin_amdgcn_perm(r2, __builtin_amdgcn_perm(r1, r0, sel01), sel2);
}

// The same for the four channels of a column at once, in six permutes instead of eight: the first two rows are
// interleaved pairwise (channels 0 and 1 in one word, 2 and 3 in the other), and each channel's word then takes its
// pair and its byte of the third row.
__device__ __forceinline__ void column_words(uint32_t r0, uint32_t r1, uint32_t r2, uint32_t (&out)[4]) {
    const uint32_t t01 = __builtin_amdgcn_perm(r1, r0, 0x05010400u);  // r0.b0 r1.b0 r0.b1 r1.b1
    const uint32_t t23 = __builtin_amdgcn_perm(r1, r0, 0x07030602u);  // r0.b2 r1.b2 r0.b3 r1.b3
    out[0] = __builtin_amdgcn_perm(r2, t01, 0x0c040100u);
    out[1] = __builtin_amdgcn_perm(r2, t01, 0x0c050302u);
    out[2] = __builtin_amdgcn_perm(r2, t23, 0x0c060100u);
    out[3] = __builtin_amdgcn_perm(r2, t23, 0x0c070302u);
}

// The same tile with 8-bit dot products, for weights whose differences w - zp_w all fit int8 (per-tensor
// requantization): activations as a - 128, the three vertical taps of a channel and column gathered into one word
// once and used by every output that touches the column (v_dot4_i32_i8 against the column's three weights), the
// term (zp_in - 128) * sum (w - zp_w) folded into the bias.  Six instructions per output for the taps instead of ten.
// TW output pixels per thread: four, or eight for stride 1 on rows that are whole tiles of eight (the column words and
// the index arithmetic are then shared by twice as many outputs).
// PC: one multiplier and shift per channel, all inside the single-shift form's range (p.rq.fast != 0).
// FOLD: weights of any range.  The products are then unsigned dot products of the raw bytes a and w, and
//     sum (a - za)(w - zw) = sum a w - zw * sum a - za * sum w + 9 za zw
// with the last two terms folded into the bias and sum a (nine taps, those outside the image reading za) taken from
// per-column sums that neighbouring outputs share: one more dot product per column and channel.  p.zp_w is then the
// zero point of the uint8 values being multiplied (int8 weights: + 128).
// D: the dilation (stride 1 only).  2 or 4: the tile's outputs j and j + D share input columns, so it reads
// TW + 2 D columns.  0: any dilation, read from the problem; no column is shared then and the tile reads three groups of
// TW adjacent columns, one per kernel column (what remains shared is the index arithmetic, the weights and the
// border tests).
__device__ __forceinline__ int udot4(uint32_t a, uint32_t b, int acc) { return (int)__builtin_amdgcn_udot4(a, b, (uint32_t)acc, false); }

template <int S, bool FLIP, int TW = 4, bool PC = false, bool FOLD = false, int D = 1>
__global__ __launch_bounds__(256) void dw3x3_nhwc_tile4_dot4_kernel(const DwProblem p, const uint32_t total, const int tiles_x,
                                                                    const FastDiv div_cq, const FastDiv div_tiles, const FastDiv div_ho) {
    static_assert(D == 1 || S == 1, "dilated tiles are stride 1");
    constexpr int IW = D ? (TW - 1) * S + 2 * D + 1 : 3 * TW;
    const int dil = D ? D : p.dil_w;
    // tile column x lies this many pixels right of the tile's first input column; output j's tap kx reads tile column col_of(j, kx)
    auto x_offset = [&](int x) { return D ? x : (x / TW) * dil + (x % TW); };
    auto col_of = [](int j, int kx) { return D ? j * S + kx * D : kx * TW + j; };
    const uint32_t idx = xcd_contiguous_block() * 256u + threadIdx.x;
    if (idx >= total) return;
    const uint32_t cq_count = (uint32_t)p.c >> 2;
    uint32_t r = fastdiv(idx, div_cq);
    const uint32_t cq = idx - r * cq_count;
    const uint32_t r2 = fastdiv(r, div_tiles);
    const int tx = (int)(r - r2 * (uint32_t)tiles_x);
    const uint32_t img = fastdiv(r2, div_ho);
    const int oy = (int)(r2 - img * (uint32_t)p.ho);
    const int ox0 = tx * TW;
    const int iy0 = oy * S - p.pad_t, ix0 = ox0 * S - p.pad_l;
    // what a tap outside the image reads, as an operand of the form in use: the input zero point (FOLD) or that minus 128
    const uint32_t fill = ((uint32_t)p.zp_in * 0x01010101u) ^ (FOLD ? 0u : 0x80808080u);
    // uint8 tensors hold a, int8 tensors a - 128: the signed form wants a - 128, the unsigned one a
    constexpr bool flip_loaded = FOLD ? FLIP : !FLIP;
    const uint32_t base = img * (uint32_t)(p.h * p.w_ * p.c) + cq * 4u;

    // (row pitch and pixel offsets stay below 2^24, which the launcher checks: 24-bit multiplies run at full rate,
    // 32-bit ones at a quarter of it)
    const int row_pitch = p.w_ * p.c;
    uint32_t in[3][IW];
    const bool inside = iy0 >= 0 && iy0 + 2 * dil < p.h && ix0 >= 0 && ix0 + x_offset(IW - 1) < p.w_;
    if (__builtin_amdgcn_ballot_w64(!inside) == 0) {
        // every window of the wave lies inside the image (most waves): no clamps, no selects, offsets that differ
        // between the loads by wave-uniform amounts; a wave with one window on the border takes the general path whole
        const uint8_t *src = p.in + (base + (uint32_t)__mul24(iy0, row_pitch) + (uint32_t)__mul24(ix0, p.c));
#pragma unroll
        for (int ky = 0; ky < 3; ++ky)
#pragma unroll
            for (int x = 0; x < IW; ++x) {
                const uint32_t v = *reinterpret_cast<const uint32_t *>(src + (uint32_t)(ky * dil * row_pitch + x_offset(x) * p.c));
                in[ky][x] = flip_loaded ? v ^ 0x80808080u : v;
            }
    } else {
        uint32_t col_off[IW];
        bool col_ok[IW];
#pragma unroll
        for (int x = 0; x < IW; ++x) {
            const int ix = ix0 + x_offset(x);
            col_ok[x] = (unsigned)ix < (unsigned)p.w_;
            const int ixc = ix < 0 ? 0 : (ix >= p.w_ ? p.w_ - 1 : ix);
            col_off[x] = base + (uint32_t)__mul24(ixc, p.c);
        }
#pragma unroll
        for (int ky = 0; ky < 3; ++ky) {
            const int iy = iy0 + ky * dil;
            const bool row_ok = (unsigned)iy < (unsigned)p.h;
            const int iyc = iy < 0 ? 0 : (iy >= p.h ? p.h - 1 : iy);
            const uint32_t row_off = (uint32_t)__mul24(iyc, row_pitch);
#pragma unroll
            for (int x = 0; x < IW; ++x) {
                const uint32_t v = *reinterpret_cast<const uint32_t *>(p.in + (row_off + col_off[x]));
                in[ky][x] = row_ok && col_ok[x] ? (flip_loaded ? v ^ 0x80808080u : v) : fill;
            }
        }
    }
    int4 wk[3];
#pragma unroll
    for (int kx = 0; kx < 3; ++kx) wk[kx] = *reinterpret_cast<const int4 *>((FOLD ? p.w_fold : p.w_trip) + ((uint32_t)kx * (uint32_t)p.cout + cq * 4u));
    const int4 b4 = *reinterpret_cast<const int4 *>((FOLD ? p.bias_fold : p.bias_trip) + cq * 4u);
    uint32_t col[IW][4];
    int cs[FOLD ? IW : 1][4];  // FOLD: sum of the column's three bytes
#pragma unroll
    for (int x = 0; x < IW; ++x) {
        column_words(in[0][x], in[1][x], in[2][x], col[x]);
        if constexpr (FOLD) {
#pragma unroll
            for (int c = 0; c < 4; ++c) cs[x][c] = udot4(col[x][c], 0x00010101u, 0);
        }
    }
    uint8_t *dst = p.out + (((img * (uint32_t)p.ho + (uint32_t)oy) * (uint32_t)p.wo + (uint32_t)ox0) * (uint32_t)p.cout + cq * 4u);
    const RequantDev rq = p.rq;
    const ChannelQuad quad = load_channel_quad<PC>(rq, cq * 4u);
#pragma unroll
    for (int j = 0; j < TW; ++j) {
        int acc0 = b4.x, acc1 = b4.y, acc2 = b4.z, acc3 = b4.w;
#pragma unroll
        for (int kx = 0; kx < 3; ++kx) {
            if constexpr (FOLD) {
                acc0 = udot4(col[col_of(j, kx)][0], (uint32_t)wk[kx].x, acc0);
                acc1 = udot4(col[col_of(j, kx)][1], (uint32_t)wk[kx].y, acc1);
                acc2 = udot4(col[col_of(j, kx)][2], (uint32_t)wk[kx].z, acc2);
                acc3 = udot4(col[col_of(j, kx)][3], (uint32_t)wk[kx].w, acc3);
            } else {
                acc0 = __builtin_amdgcn_sdot4((int)col[col_of(j, kx)][0], wk[kx].x, acc0, false);
                acc1 = __builtin_amdgcn_sdot4((int)col[col_of(j, kx)][1], wk[kx].y, acc1, false);
                acc2 = __builtin_amdgcn_sdot4((int)col[col_of(j, kx)][2], wk[kx].z, acc2, false);
                acc3 = __builtin_amdgcn_sdot4((int)col[col_of(j, kx)][3], wk[kx].w, acc3, false);
            }
        }
        if constexpr (FOLD) {
            // (nine bytes times a zero point of at most 383: a 24-bit multiply-add)
            acc0 += __mul24(-p.zp_w, cs[col_of(j, 0)][0] + cs[col_of(j, 1)][0] + cs[col_of(j, 2)][0]);
            acc1 += __mul24(-p.zp_w, cs[col_of(j, 0)][1] + cs[col_of(j, 1)][1] + cs[col_of(j, 2)][1]);
            acc2 += __mul24(-p.zp_w, cs[col_of(j, 0)][2] + cs[col_of(j, 1)][2] + cs[col_of(j, 2)][2]);
            acc3 += __mul24(-p.zp_w, cs[col_of(j, 0)][3] + cs[col_of(j, 1)][3] + cs[col_of(j, 2)][3]);
        }
        uint32_t o = PC ? requant4_channel_fast(acc0, acc1, acc2, acc3, rq, quad) : requant4<false>(acc0, acc1, acc2, acc3, rq, quad);
        if (FLIP) o ^= 0x80808080u;
        if (ox0 + j < p.wo) *reinterpret_cast<uint32_t *>(dst + (uint32_t)j * (uint32_t)p.cout) = o;
    }
}

// 5x5 and 7x7 kernels with the same tile (four adjacent channels of four horizontally adjacent output pixels per thread)
// and the unsigned dot-product form.  The tile's input columns are walked one at a time: a column's K words (one per
// row, four channels each) are turned into two words per channel holding its vertical taps 0..3 and 4..K-1, whose dot
// products with the kernel column kx = x - j S go to every output j of the tile that the column lies under, and whose
// byte sum goes to those outputs' zero-point term.  A kernel column's two weight words are read when the walk first
// needs them and are used by four consecutive (stride 2: every other) input columns.  Replaces the one-pixel kernel's
// K*K 16-bit multiply-adds per output by 2 K dot products shared between the tile's pixels.
template <int K, int S, bool FLIP>
__global__ __launch_bounds__(256) void dwkxk_nhwc_tile4_kernel(const DwProblem p, const uint32_t total, const int tiles_x, const FastDiv div_cq,
                                                               const FastDiv div_tiles, const FastDiv div_ho) {
    static_assert(K == 5 || K == 7, "two words per kernel column: four taps and the other one or three");
    constexpr int TW = 4, IW = (TW - 1) * S + K;
    const uint32_t idx = xcd_contiguous_block() * 256u + threadIdx.x;
    if (idx >= total) return;
    const uint32_t cq_count = (uint32_t)p.c >> 2;
    uint32_t r = fastdiv(idx, div_cq);
    const uint32_t cq = idx - r * cq_count;
    const uint32_t r2 = fastdiv(r, div_tiles);
    const int tx = (int)(r - r2 * (uint32_t)tiles_x);
    const uint32_t img = fastdiv(r2, div_ho);
    const int oy = (int)(r2 - img * (uint32_t)p.ho);
    const int ox0 = tx * TW;
    const int iy0 = oy * S - p.pad_t, ix0 = ox0 * S - p.pad_l;
    const uint32_t fill = (uint32_t)p.zp_in * 0x01010101u;
    const uint32_t flip_word = FLIP ? 0x80808080u : 0u;  // int8 tensors: the bytes as uint8 values
    const uint32_t base = img * (uint32_t)(p.h * p.w_ * p.c) + cq * 4u;
    const int row_pitch = p.w_ * p.c;
    const bool inside = iy0 >= 0 && iy0 + K - 1 < p.h && ix0 >= 0 && ix0 + IW - 1 < p.w_;
    const bool all_inside = __builtin_amdgcn_ballot_w64(!inside) == 0;
    const uint8_t *src = p.in + (base + (uint32_t)__mul24(iy0 < 0 ? 0 : iy0, row_pitch) + (uint32_t)__mul24(ix0 < 0 ? 0 : ix0, p.c));
    uint32_t row_off[K];
    bool row_ok[K];
#pragma unroll
    for (int ky = 0; ky < K; ++ky) {
        const int iy = iy0 + ky;
        row_ok[ky] = (unsigned)iy < (unsigned)p.h;
        const int iyc = iy < 0 ? 0 : (iy >= p.h ? p.h - 1 : iy);
        row_off[ky] = base + (uint32_t)__mul24(iyc, row_pitch);
    }
    const int4 b4 = *reinterpret_cast<const int4 *>(p.bias_foldk + cq * 4u);
    int acc[TW][4], csum[TW][4];
#pragma unroll
    for (int j = 0; j < TW; ++j) {
        acc[j][0] = b4.x;
        acc[j][1] = b4.y;
        acc[j][2] = b4.z;
        acc[j][3] = b4.w;
#pragma unroll
        for (int c = 0; c < 4; ++c) csum[j][c] = 0;
    }
    auto load_column = [&](int x, uint32_t (&rows)[K]) {
        if (all_inside) {
#pragma unroll
            for (int ky = 0; ky < K; ++ky) rows[ky] = *reinterpret_cast<const uint32_t *>(src + (uint32_t)(ky * row_pitch + x * p.c)) ^ flip_word;
        } else {
            const int ix = ix0 + x;
            const bool col_ok = (unsigned)ix < (unsigned)p.w_;
            const uint32_t col_off = (uint32_t)__mul24(ix < 0 ? 0 : (ix >= p.w_ ? p.w_ - 1 : ix), p.c);
#pragma unroll
            for (int ky = 0; ky < K; ++ky) {
                const uint32_t v = *reinterpret_cast<const uint32_t *>(p.in + (row_off[ky] + col_off)) ^ flip_word;
                rows[ky] = row_ok[ky] && col_ok ? v : fill;
            }
        }
    };
    // The walk is fenced column by column: left alone the compiler requests every column and every weight word at the
    // top (170 registers for 7x7, two waves per SIMD); fenced, a column's words and the weights of the kernel column
    // that enters with it are requested one column ahead.
    int4 wk[K][2];
    auto load_weights = [&](int kx) {
        wk[kx][0] = *reinterpret_cast<const int4 *>(p.w_foldk + ((uint32_t)(kx * 2) * (uint32_t)p.cout + cq * 4u));
        wk[kx][1] = *reinterpret_cast<const int4 *>(p.w_foldk + ((uint32_t)(kx * 2 + 1) * (uint32_t)p.cout + cq * 4u));
    };
    uint32_t ahead[K];
    load_column(0, ahead);
    load_weights(0);
#pragma unroll
    for (int x = 0; x < IW; ++x) {
        uint32_t rows[K];
#pragma unroll
        for (int ky = 0; ky < K; ++ky) rows[ky] = ahead[ky];
        if (x + 1 < K) load_weights(x + 1);  // the kernel column that enters the walk at the next input column
        if (x + 1 < IW) load_column(x + 1, ahead);
        __builtin_amdgcn_sched_barrier(0);
        // rows 0..3: a 4 x 4 byte transpose; the rest: the three-row gather of the 3x3 kernel, or single bytes
        uint32_t lo[4], hi[4];
        {
            const uint32_t t0 = __builtin_amdgcn_perm(rows[1], rows[0], 0x05010400u), t1 = __builtin_amdgcn_perm(rows[1], rows[0], 0x07030602u);
            const uint32_t u0 = __builtin_amdgcn_perm(rows[3], rows[2], 0x05010400u), u1 = __builtin_amdgcn_perm(rows[3], rows[2], 0x07030602u);
            lo[0] = __builtin_amdgcn_perm(u0, t0, 0x05040100u);
            lo[1] = __builtin_amdgcn_perm(u0, t0, 0x07060302u);
            lo[2] = __builtin_amdgcn_perm(u1, t1, 0x05040100u);
            lo[3] = __builtin_amdgcn_perm(u1, t1, 0x07060302u);
        }
        if constexpr (K == 7) {
            column_words(rows[4], rows[5], rows[6], hi);
        } else {
            hi[0] = rows[4] & 0xFFu;
            hi[1] = (rows[4] >> 8) & 0xFFu;
            hi[2] = (rows[4] >> 16) & 0xFFu;
            hi[3] = rows[4] >> 24;
        }
        int cs[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) cs[c] = udot4(hi[c], 0x01010101u, udot4(lo[c], 0x01010101u, 0));
#pragma unroll
        for (int j = 0; j < TW; ++j) {
            const int kx = x - j * S;
            if (kx < 0 || kx >= K) continue;
            acc[j][0] = udot4(hi[0], (uint32_t)wk[kx][1].x, udot4(lo[0], (uint32_t)wk[kx][0].x, acc[j][0]));
            acc[j][1] = udot4(hi[1], (uint32_t)wk[kx][1].y, udot4(lo[1], (uint32_t)wk[kx][0].y, acc[j][1]));
            acc[j][2] = udot4(hi[2], (uint32_t)wk[kx][1].z, udot4(lo[2], (uint32_t)wk[kx][0].z, acc[j][2]));
            acc[j][3] = udot4(hi[3], (uint32_t)wk[kx][1].w, udot4(lo[3], (uint32_t)wk[kx][0].w, acc[j][3]));
#pragma unroll
            for (int c = 0; c < 4; ++c) csum[j][c] += cs[c];
        }
    }
    uint8_t *dst = p.out + (((img * (uint32_t)p.ho + (uint32_t)oy) * (uint32_t)p.wo + (uint32_t)ox0) * (uint32_t)p.cout + cq * 4u);
    const RequantDev rq = p.rq;
    const ChannelQuad quad{};
#pragma unroll
    for (int j = 0; j < TW; ++j) {
        // (K * K bytes times a zero point of at most 383: a 24-bit multiply-add)
        const int a0 = acc[j][0] + __mul24(-p.zp_w, csum[j][0]), a1 = acc[j][1] + __mul24(-p.zp_w, csum[j][1]);
        const int a2 = acc[j][2] + __mul24(-p.zp_w, csum[j][2]), a3 = acc[j][3] + __mul24(-p.zp_w, csum[j][3]);
        uint32_t o = requant4<false>(a0, a1, a2, a3, rq, quad);
        if (FLIP) o ^= 0x80808080u;
        if (ox0 + j < p.wo) *reinterpret_cast<uint32_t *>(dst + (uint32_t)j * (uint32_t)p.cout) = o;
    }
}

// One output element per thread; any depth multiplier, dilation, channel count.
// NHWC = true: channel fastest.  NHWC = false: planar NCHW, x fastest.
template <bool NHWC>
__global__ __launch_bounds__(256) void dw_scalar_kernel(const DwProblem p, const long total) {
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    int oc, ox, oy, img;
    if (total < (1l << 31)) {  // (uniform) 32-bit divisions: a fraction of the 64-bit ones' instructions
        const uint32_t i = (uint32_t)idx, d0 = (uint32_t)(NHWC ? p.cout : p.wo), d2 = (uint32_t)(NHWC ? p.ho : p.cout);
        const uint32_t d1 = (uint32_t)(NHWC ? p.wo : p.ho);
        const uint32_t r0 = i / d0, r1 = r0 / d1, r2 = r1 / d2;
        const int f0 = (int)(i - r0 * d0), f1 = (int)(r0 - r1 * d1), f2 = (int)(r1 - r2 * d2);
        img = (int)r2;
        if (NHWC)
            oc = f0, ox = f1, oy = f2;
        else
            ox = f0, oy = f1, oc = f2;
    } else if (NHWC) {
        oc = (int)(idx % p.cout);
        long r = idx / p.cout;
        ox = (int)(r % p.wo);
        r /= p.wo;
        oy = (int)(r % p.ho);
        img = (int)(r / p.ho);
    } else {
        ox = (int)(idx % p.wo);
        long r = idx / p.wo;
        oy = (int)(r % p.ho);
        r /= p.ho;
        oc = (int)(r % p.cout);
        img = (int)(r / p.cout);
    }
    const int ic = oc / p.dm;
    int32_t acc = p.bias ? p.bias[oc] : 0;
    const int iy0 = oy * p.stride_h - p.pad_t, ix0 = ox * p.stride_w - p.pad_l;
    for (int ky = 0; ky < p.kh; ++ky) {
        const int iy = iy0 + ky * p.dil_h;
        if ((unsigned)iy >= (unsigned)p.h) continue;
        for (int kx = 0; kx < p.kw; ++kx) {
            const int ix = ix0 + kx * p.dil_w;
            if ((unsigned)ix >= (unsigned)p.w_) continue;
            const size_t a_idx = NHWC ? (((size_t)img * p.h + iy) * p.w_ + ix) * p.c + ic
                                      : (((size_t)img * p.c + ic) * p.h + iy) * p.w_ + ix;
            const int32_t a = (int32_t)(p.in[a_idx] ^ (p.io_flip & 0xFFu)) - p.zp_in;
            const uint8_t raw = p.w[((size_t)oc * p.kh + ky) * p.kw + kx];
            const int32_t w = (p.w_signed ? (int32_t)(int8_t)raw : (int32_t)raw) - p.zp_w;
            acc += a * w;
        }
    }
    p.out[idx] = (uint8_t)((p.rq.pc_multiplier ? requant_u8_channel(acc, p.rq.pc_multiplier[oc], p.rq.pc_shift[oc], p.rq)
                                                : requant_u8(acc, p.rq)) ^ (p.io_flip & 0xFFu));
}

__global__ void dw_pack_kernel(const uint8_t *w, const int32_t *bias, int32_t *w_pair, int32_t *bias_folded, int32_t cout,
                               int32_t taps, int32_t zp_in, int32_t zp_w, int32_t w_signed) {
    const int oc = blockIdx.x * blockDim.x + threadIdx.x;
    if (oc >= cout) return;
    int32_t sum = 0;
    const int pairs = (taps + 1) >> 1;
    for (int pr = 0; pr < pairs; ++pr) {
        auto value = [&](int t) {
            const uint8_t raw = w[(size_t)oc * taps + t];
            return (w_signed ? (int32_t)(int8_t)raw : (int32_t)raw) - zp_w;
        };
        const int32_t lo = value(2 * pr);
        const int32_t hi = 2 * pr + 1 < taps ? value(2 * pr + 1) : 0;
        sum += lo + hi;
        w_pair[(size_t)pr * cout + oc] = (int32_t)(((uint32_t)lo & 0xFFFFu) | ((uint32_t)hi << 16));
    }
    bias_folded[oc] = (bias ? bias[oc] : 0) - zp_in * sum;
}

// 3x3 weights [cout][9] -> w_trip[kx][cout]: the three vertical taps (w - zp_w, each known to fit int8) of column kx
// in bytes 0..2; bias_trip[c] = bias - (zp_in - 128) * sum (w - zp_w)
__global__ void dw_pack_trip_kernel(const uint8_t *w, const int32_t *bias, int32_t *w_trip, int32_t *bias_trip, int32_t cout,
                                    int32_t zp_in, int32_t zp_w, int32_t w_signed) {
    const int oc = blockIdx.x * blockDim.x + threadIdx.x;
    if (oc >= cout) return;
    int32_t sum = 0;
    for (int kx = 0; kx < 3; ++kx) {
        uint32_t word = 0;
        for (int ky = 0; ky < 3; ++ky) {
            const uint8_t raw = w[(size_t)oc * 9 + ky * 3 + kx];
            const int32_t v = (w_signed ? (int32_t)(int8_t)raw : (int32_t)raw) - zp_w;
            sum += v;
            word |= ((uint32_t)v & 255u) << (8 * ky);
        }
        w_trip[(size_t)kx * cout + oc] = (int32_t)word;
    }
    bias_trip[oc] = (bias ? bias[oc] : 0) - (zp_in - 128) * sum;
}

// 3x3 weights [cout][9] -> w_fold[kx][cout]: the three vertical taps of column kx as the uint8 values the unsigned
// form multiplies (int8 weights: byte + 128, `zp_w` being their zero point + 128) in bytes 0..2;
// bias_fold[c] = bias - zp_in * sum w + 9 * zp_in * zp_w
__global__ void dw_pack_fold_kernel(const uint8_t *w, const int32_t *bias, int32_t *w_fold, int32_t *bias_fold, int32_t cout,
                                    int32_t zp_in, int32_t zp_w, int32_t w_signed) {
    const int oc = blockIdx.x * blockDim.x + threadIdx.x;
    if (oc >= cout) return;
    int32_t sum = 0;
    for (int kx = 0; kx < 3; ++kx) {
        uint32_t word = 0;
        for (int ky = 0; ky < 3; ++ky) {
            const uint32_t v = (uint32_t)w[(size_t)oc * 9 + ky * 3 + kx] ^ (w_signed ? 0x80u : 0u);
            sum += (int32_t)v;
            word |= v << (8 * ky);
        }
        w_fold[(size_t)kx * cout + oc] = (int32_t)word;
    }
    bias_fold[oc] = (bias ? bias[oc] : 0) - zp_in * sum + 9 * zp_in * zp_w;
}

// K x K weights [cout][K*K] -> w_foldk[kx][2][cout]: the vertical taps 0..3 and 4..K-1 of column kx as uint8 bytes (int8
// weights: byte + 128, `zp_w` being their zero point + 128); bias_foldk[c] = bias - zp_in * sum w + K K zp_in zp_w
__global__ void dw_pack_foldk_kernel(const uint8_t *w, const int32_t *bias, int32_t *w_foldk, int32_t *bias_foldk, int32_t cout, int32_t k,
                                     int32_t zp_in, int32_t zp_w, int32_t w_signed) {
    const int oc = blockIdx.x * blockDim.x + threadIdx.x;
    if (oc >= cout) return;
    int32_t sum = 0;
    for (int kx = 0; kx < k; ++kx) {
        uint32_t word[2] = {0, 0};
        for (int ky = 0; ky < k; ++ky) {
            const uint32_t v = (uint32_t)w[(size_t)oc * k * k + ky * k + kx] ^ (w_signed ? 0x80u : 0u);
            sum += (int32_t)v;
            word[ky >> 2] |= v << (8 * (ky & 3));
        }
        w_foldk[(size_t)(kx * 2) * cout + oc] = (int32_t)word[0];
        w_foldk[(size_t)(kx * 2 + 1) * cout + oc] = (int32_t)word[1];
    }
    bias_foldk[oc] = (bias ? bias[oc] : 0) - zp_in * sum + k * k * zp_in * zp_w;
}

}  // namespace

int launch_dw_pack_foldk(const uint8_t *w, const int32_t *bias, int32_t *w_foldk, int32_t *bias_foldk, int32_t cout, int32_t k,
                         int32_t zp_in, int32_t zp_w_u8, int32_t w_signed, hipStream_t stream) {
    if (cout <= 0) return EH_OK;
    hipLaunchKernelGGL(dw_pack_foldk_kernel, dim3((cout + 127) / 128), dim3(128), 0, stream, w, bias, w_foldk, bias_foldk, cout, k, zp_in,
                       zp_w_u8, w_signed);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

int launch_dw_pack_fold(const uint8_t *w, const int32_t *bias, int32_t *w_fold, int32_t *bias_fold, int32_t cout, int32_t zp_in,
                        int32_t zp_w_u8, int32_t w_signed, hipStream_t stream) {
    if (cout <= 0) return EH_OK;
    hipLaunchKernelGGL(dw_pack_fold_kernel, dim3((cout + 127) / 128), dim3(128), 0, stream, w, bias, w_fold, bias_fold, cout, zp_in,
                       zp_w_u8, w_signed);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

int launch_dw_pack(const uint8_t *w, const int32_t *bias, int32_t *w_pair, int32_t *bias_folded, int32_t cout,
                   int32_t taps, int32_t zp_in, int32_t zp_w, int32_t w_signed, hipStream_t stream) {
    if (cout <= 0) return EH_OK;
    hipLaunchKernelGGL(dw_pack_kernel, dim3((cout + 127) / 128), dim3(128), 0, stream, w, bias, w_pair, bias_folded, cout,
                       taps, zp_in, zp_w, w_signed);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

int launch_dw_pack_trip(const uint8_t *w, const int32_t *bias, int32_t *w_trip, int32_t *bias_trip, int32_t cout, int32_t zp_in,
                        int32_t zp_w, int32_t w_signed, hipStream_t stream) {
    if (cout <= 0) return EH_OK;
    hipLaunchKernelGGL(dw_pack_trip_kernel, dim3((cout + 127) / 128), dim3(128), 0, stream, w, bias, w_trip, bias_trip, cout, zp_in, zp_w,
                       w_signed);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

static long pairs_of(const DwProblem &p) { return ((long)p.kh * p.kw + 1) / 2; }

int launch_dwconv_nhwc(const DwProblem &caller_p, hipStream_t stream) {
    DwProblem p = caller_p;
    const bool pc_two_step = p.rq.pc_multiplier != nullptr && !p.rq.fast;
    if (p.w_trip || pc_two_step) p.w_fold = nullptr;  // the signed form where it applies; per-channel pairs outside the single-shift range use the 16-bit kernel
    const long outs = (long)p.n * p.ho * p.wo * p.cout;
    if (outs <= 0) return EH_OK;
    const bool vec = p.dm == 1 && (p.c & 3) == 0 && (reinterpret_cast<uintptr_t>(p.in) & 3) == 0 &&
                     (reinterpret_cast<uintptr_t>(p.out) & 3) == 0;
    // (the dot product kernels index rows and pixels with 24-bit multiplies)
    const bool dot4_form = (p.w_trip || p.w_fold) && (p.rq.pc_multiplier == nullptr || p.rq.fast) && (long)p.w_ * p.c < (1l << 23) && p.h < (1 << 23);
    const bool dilated = p.dil_h > 1 && p.dil_h == p.dil_w && p.stride_h == 1 && dot4_form && (long)p.dil_h * p.w_ * p.c < (1l << 22);
    const bool tile3x3 = vec && p.kh == 3 && p.kw == 3 && ((p.dil_h == 1 && p.dil_w == 1) || dilated) && p.stride_h == p.stride_w &&
                         (p.stride_h == 1 || p.stride_h == 2) && (size_t)p.n * p.h * p.w_ * p.c < (1ull << 31) &&
                         (size_t)p.n * p.ho * p.wo * p.cout < (1ull << 31);
    const bool tile_kxk = vec && p.w_foldk != nullptr && p.kh == p.kw && (p.kh == 5 || p.kh == 7) && p.dil_h == 1 && p.dil_w == 1 && p.dm == 1 &&
                          (p.c & 3) == 0 && p.stride_h == p.stride_w && (p.stride_h == 1 || p.stride_h == 2) && p.rq.pc_multiplier == nullptr &&
                          p.pad_t >= 0 && p.pad_l >= 0 && (size_t)p.n * p.h * p.w_ * p.c < (1ull << 31) &&
                          (size_t)p.n * p.ho * p.wo * p.cout < (1ull << 31) && (long)p.w_ * p.c < (1l << 23) && p.h < (1 << 23);
    if (tile_kxk) {
        DwProblem q = p;
        q.zp_w += q.w_signed ? 128 : 0;  // zero point of the uint8 values the unsigned form multiplies
        const int tiles_x = (q.wo + 3) / 4;
        const long total = (long)q.n * q.ho * tiles_x * (q.c >> 2);
        EH_REQUIRE(total < (1l << 31), "depthwise: grid too large");
        const long blocks = (total + 255) / 256;
        const FastDiv d_cq = make_fastdiv((uint32_t)(q.c >> 2)), d_t = make_fastdiv((uint32_t)tiles_x), d_ho = make_fastdiv((uint32_t)q.ho);
        const bool flip = q.io_flip != 0;
        auto pick = [&](auto k_c, auto s_c) {
            constexpr int K = decltype(k_c)::value, S = decltype(s_c)::value;
            return flip ? dwkxk_nhwc_tile4_kernel<K, S, true> : dwkxk_nhwc_tile4_kernel<K, S, false>;
        };
        using one = std::integral_constant<int, 1>;
        using two = std::integral_constant<int, 2>;
        auto kernel = q.kh == 5 ? (q.stride_h == 1 ? pick(std::integral_constant<int, 5>{}, one{}) : pick(std::integral_constant<int, 5>{}, two{}))
                                : (q.stride_h == 1 ? pick(std::integral_constant<int, 7>{}, one{}) : pick(std::integral_constant<int, 7>{}, two{}));
        hipLaunchKernelGGL(kernel, dim3((unsigned)((blocks + 7) / 8 * 8)), dim3(256), 0, stream, q, (uint32_t)total, tiles_x, d_cq, d_t, d_ho);
        EH_HIP(hipGetLastError());
        return EH_OK;
    }
    if (tile3x3) {
        // zero point of the uint8 values the unsigned form multiplies (only here: the one-output-per-thread kernel reads
        // the weights as the caller quantized them)
        if (p.w_fold) p.zp_w += p.w_signed ? 128 : 0;
        const int tiles_x = (p.wo + 3) / 4;
        const long total = (long)p.n * p.ho * tiles_x * (p.c >> 2);
        const long blocks = (total + 255) / 256;
        EH_REQUIRE(total < (1l << 31), "depthwise: grid too large");
        const FastDiv d_cq = make_fastdiv((uint32_t)(p.c >> 2)), d_t = make_fastdiv((uint32_t)tiles_x), d_ho = make_fastdiv((uint32_t)p.ho);
        // per-channel pairs and int8 tensors are compile-time variants: the plain uint8 kernel pays for neither
        const bool pc = p.rq.pc_multiplier != nullptr, flip = p.io_flip != 0;
        auto pick = [&](auto stride_c) {
            constexpr int S = decltype(stride_c)::value;
            return pc ? (flip ? dw3x3_nhwc_tile4_kernel<S, true, true> : dw3x3_nhwc_tile4_kernel<S, true, false>)
                      : (flip ? dw3x3_nhwc_tile4_kernel<S, false, true> : dw3x3_nhwc_tile4_kernel<S, false, false>);
        };
        auto kernel = p.stride_h == 1 ? pick(std::integral_constant<int, 1>{}) : pick(std::integral_constant<int, 2>{});
        // 8-bit dot products: the signed form where every w - zp_w fits int8, else the unsigned form for any weights
        const bool fold = p.w_trip == nullptr;
        auto pick_dot4 = [&](auto s_tag, auto tw_tag) {
            constexpr int S = decltype(s_tag)::value, TW = decltype(tw_tag)::value;
            if (fold)
                return pc ? (flip ? dw3x3_nhwc_tile4_dot4_kernel<S, true, TW, true, true> : dw3x3_nhwc_tile4_dot4_kernel<S, false, TW, true, true>)
                          : (flip ? dw3x3_nhwc_tile4_dot4_kernel<S, true, TW, false, true> : dw3x3_nhwc_tile4_dot4_kernel<S, false, TW, false, true>);
            return pc ? (flip ? dw3x3_nhwc_tile4_dot4_kernel<S, true, TW, true> : dw3x3_nhwc_tile4_dot4_kernel<S, false, TW, true>)
                      : (flip ? dw3x3_nhwc_tile4_dot4_kernel<S, true, TW, false> : dw3x3_nhwc_tile4_dot4_kernel<S, false, TW, false>);
        };
        using tw4 = std::integral_constant<int, 4>;
        const bool dot4 = dot4_form;
        if (p.dil_h > 1) {
            // dilated, stride 1: the tiles that share columns for dilations 2 and 4, the three-group tile for the rest
            auto pick_dilated = [&](auto d_tag) {
                constexpr int D = decltype(d_tag)::value;
                if (fold)
                    return pc ? (flip ? dw3x3_nhwc_tile4_dot4_kernel<1, true, 4, true, true, D> : dw3x3_nhwc_tile4_dot4_kernel<1, false, 4, true, true, D>)
                              : (flip ? dw3x3_nhwc_tile4_dot4_kernel<1, true, 4, false, true, D> : dw3x3_nhwc_tile4_dot4_kernel<1, false, 4, false, true, D>);
                return pc ? (flip ? dw3x3_nhwc_tile4_dot4_kernel<1, true, 4, true, false, D> : dw3x3_nhwc_tile4_dot4_kernel<1, false, 4, true, false, D>)
                          : (flip ? dw3x3_nhwc_tile4_dot4_kernel<1, true, 4, false, false, D> : dw3x3_nhwc_tile4_dot4_kernel<1, false, 4, false, false, D>);
            };
            kernel = p.dil_h == 2   ? pick_dilated(std::integral_constant<int, 2>{})
                     : p.dil_h == 4 ? pick_dilated(std::integral_constant<int, 4>{})
                                    : pick_dilated(std::integral_constant<int, 0>{});
        } else if (dot4)
            kernel = p.stride_h == 1 ? pick_dot4(std::integral_constant<int, 1>{}, tw4{}) : pick_dot4(std::integral_constant<int, 2>{}, tw4{});
        if (dot4 && p.dil_h == 1 && p.stride_h == 1 && (p.wo & 7) == 0 && total >= (1l << 20)) {
            // large stride-1 layers with rows of whole eight-pixel tiles: eight outputs per thread
            const int tiles8 = p.wo / 8;
            const long total8 = (long)p.n * p.ho * tiles8 * (p.c >> 2);
            const FastDiv d_t8 = make_fastdiv((uint32_t)tiles8);
            auto kernel8 = pick_dot4(std::integral_constant<int, 1>{}, std::integral_constant<int, 8>{});
            hipLaunchKernelGGL(kernel8, dim3((unsigned)(((total8 + 255) / 256 + 7) / 8 * 8)), dim3(256), 0, stream, p, (uint32_t)total8, tiles8, d_cq, d_t8,
                               d_ho);
            EH_HIP(hipGetLastError());
            return EH_OK;
        }
        hipLaunchKernelGGL(kernel, dim3((unsigned)((blocks + 7) / 8 * 8)), dim3(256), 0, stream, p, (uint32_t)total, tiles_x, d_cq, d_t, d_ho);
    } else if (vec) {
        const long total = outs / 4;
        const long blocks = (total + 255) / 256;
        EH_REQUIRE(blocks < (1l << 31), "depthwise: grid too large");
        const bool small = (size_t)p.n * p.h * p.w_ * p.c < (1ull << 31) && outs < (1l << 31) && (size_t)pairs_of(p) * p.cout < (1ull << 30);
        const FastDiv d_cq = make_fastdiv((uint32_t)(p.c >> 2)), d_wo = make_fastdiv((uint32_t)p.wo), d_ho = make_fastdiv((uint32_t)p.ho);
        const bool k3 = p.kh == 3 && p.kw == 3;
        auto kernel = k3 ? (small ? dw_nhwc_vec4_kernel<3, 3, true> : dw_nhwc_vec4_kernel<3, 3, false>)
                         : (small ? dw_nhwc_vec4_kernel<0, 0, true> : dw_nhwc_vec4_kernel<0, 0, false>);
        hipLaunchKernelGGL(kernel, dim3((unsigned)((blocks + 7) / 8 * 8)), dim3(256), 0, stream, p, total, d_cq, d_wo, d_ho);
    } else {
        const long blocks = (outs + 255) / 256;
        EH_REQUIRE(blocks < (1l << 31), "depthwise: grid too large");
        hipLaunchKernelGGL((dw_scalar_kernel<true>), dim3((unsigned)blocks), dim3(256), 0, stream, p, outs);
    }
    EH_HIP(hipGetLastError());
    return EH_OK;
}

int launch_dwconv_nchw(const DwProblem &p, hipStream_t stream) {
    const long outs = (long)p.n * p.ho * p.wo * p.cout;
    if (outs <= 0) return EH_OK;
    const long blocks = (outs + 255) / 256;
    EH_REQUIRE(blocks < (1l << 31), "depthwise: grid too large");
    hipLaunchKernelGGL((dw_scalar_kernel<false>), dim3((unsigned)blocks), dim3(256), 0, stream, p, outs);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

}  // namespace eh
