// Implicit-GEMM uint8 convolution / fully-connected / deconvolution-phase kernel
// for gfx950 int8 MFMA (v_mfma_i32_32x32x32_i8), with the requantize epilogue fused.
//
// Replaces, for the uint8 path, the reference's pad + im2col + quantizedGemmBlocked
// pipeline (gpu/operators/cl_kernels/PadConvertKernels.cpp:25-167,
// ConvolutionKernels.cpp:956-1274), its direct 3x3 kernel
// (DirectConvolutionKernel.cpp:4324-4869) and the deconvolution's convBackGemmRXR +
// convertBottomDiff2 pair (DeconvolutionKernels.cpp:24-198): nothing is
// materialised in HBM between the input image and the uint8 output.
//
// Arithmetic.  MFMA multiplies signed bytes, so both operands are shifted by 128:
// a' = a - 128 (one XOR on the way into LDS), w' = w - 128 (done when the weights
// are packed).  With za = zp_in - 128 and zw = zp_w - 128,
//   sum_k (a - zp_in)(w - zp_w) = sum_k a'w' - zw * sum_k a' - za * sum_k w' + K * za * zw.
// The last two terms are per output channel and live in the folded bias; the
// second is per output pixel and is accumulated by the loader threads while the
// tile passes through their registers.  A tap outside the image reads zp_in
// (the reference pads with the input zero point, CLPadConvert.cpp:185), i.e.
// a' = za, which keeps the formula uniform; reduction-axis padding reads 128,
// i.e. a' = 0, against zero weights.
#include "eh_internal.h"

namespace eh {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

namespace {

constexpr int BK = 64;        // reduction bytes per LDS stage
constexpr int LDS_ROW = 80;   // 64 data bytes + 16 pad: 16-byte accesses from 8 consecutive rows hit 32 distinct banks
constexpr int16_t KPAD_MARK = INT16_MIN;

__device__ __forceinline__ uint4 xor128(uint4 v, uint32_t x) {
    v.x ^= x;
    v.y ^= x;
    v.z ^= x;
    v.w ^= x;
    return v;
}

__device__ __forceinline__ int sum_bytes_signed(uint4 v, int acc) {
    acc = __builtin_amdgcn_sdot4((int)v.x, 0x01010101, acc, false);
    acc = __builtin_amdgcn_sdot4((int)v.y, 0x01010101, acc, false);
    acc = __builtin_amdgcn_sdot4((int)v.z, 0x01010101, acc, false);
    acc = __builtin_amdgcn_sdot4((int)v.w, 0x01010101, acc, false);
    return acc;
}

// Loads the 16 reduction bytes [unit16*16, unit16*16+16) of one output pixel.
template <int VEC>
__device__ __forceinline__ uint4 load_a_chunk(const GemmProblem &p, int base, int iy0, int ix0, int unit16) {
    uint4 v;
    if constexpr (VEC == 16) {
        const KUnit ku = p.ktab[unit16];
        const int iy = iy0 + ku.dy, ix = ix0 + ku.dx;
        if (ku.dy == KPAD_MARK) {
            v = make_uint4(p.a_xor, p.a_xor, p.a_xor, p.a_xor);
        } else if ((unsigned)iy < (unsigned)p.h && (unsigned)ix < (unsigned)p.w) {
            v = *reinterpret_cast<const uint4 *>(p.a + (base + ku.offset));
        } else {
            v = make_uint4(p.fill, p.fill, p.fill, p.fill);
        }
    } else if constexpr (VEC == 4) {
        uint32_t d[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const KUnit ku = p.ktab[unit16 * 4 + j];
            const int iy = iy0 + ku.dy, ix = ix0 + ku.dx;
            if (ku.dy == KPAD_MARK) {
                d[j] = p.a_xor;
            } else if ((unsigned)iy < (unsigned)p.h && (unsigned)ix < (unsigned)p.w) {
                d[j] = *reinterpret_cast<const uint32_t *>(p.a + (base + ku.offset));
            } else {
                d[j] = p.fill;
            }
        }
        v = make_uint4(d[0], d[1], d[2], d[3]);
    } else {
        uint32_t d[4] = {0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const KUnit ku = p.ktab[unit16 * 16 + j];
            const int iy = iy0 + ku.dy, ix = ix0 + ku.dx;
            uint32_t b;
            if (ku.dy == KPAD_MARK) {
                b = p.a_xor & 0xFFu;
            } else if ((unsigned)iy < (unsigned)p.h && (unsigned)ix < (unsigned)p.w) {
                b = p.a[base + ku.offset];
            } else {
                b = p.fill & 0xFFu;
            }
            d[j >> 2] |= b << (8 * (j & 3));
        }
        v = make_uint4(d[0], d[1], d[2], d[3]);
    }
    return v;
}

// Workgroup tile BM x BN, WGM x WGN waves, each wave owning (BM/WGM) x (BN/WGN)
// as 32x32 MFMA tiles.  LDS holds two stages of A and B; global loads for
// stage t+1 are in flight while stage t feeds the matrix cores.
template <int BM, int BN, int WGM, int WGN, int VEC>
__global__ __launch_bounds__(WGM *WGN * 64) void igemm_u8_kernel(const GemmProblem p, const int tiles_m, const int tiles_n) {
    constexpr int THREADS = WGM * WGN * 64;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int FM = WTM / 32, FN = WTN / 32;
    constexpr int ROWS_PER_PASS = THREADS / 4;
    constexpr int A_CHUNKS = BM / ROWS_PER_PASS;
    constexpr int B_CHUNKS = BN / ROWS_PER_PASS;
    static_assert(BM % ROWS_PER_PASS == 0 && BN % ROWS_PER_PASS == 0, "tile must be a multiple of the loader pass");
    static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be made of 32x32 MFMA tiles");
    constexpr int STAGE_BYTES = (BM + BN) * LDS_ROW;
    constexpr int OUT_ROW = BN + 16;
    constexpr int LDS_BYTES = 2 * STAGE_BYTES > BM * OUT_ROW ? 2 * STAGE_BYTES : BM * OUT_ROW;

    __shared__ __align__(16) uint8_t lds[LDS_BYTES];
    __shared__ int32_t rowsum_s[BM];

    // Workgroups are dispatched round-robin over the 8 XCDs, each with its own L2.
    // Give every XCD a contiguous run of tiles, ordered m-fastest, so that the
    // workgroups that share a weight tile share an L2.
    int tile = blockIdx.x;
    const int total = tiles_m * tiles_n;
    if ((total & 7) == 0) tile = (blockIdx.x & 7) * (total >> 3) + (blockIdx.x >> 3);
    const int tm = tile % tiles_m, tn = tile / tiles_m;
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WGM, wn = wave / WGM;
    const int lrow = tid >> 2, kc = tid & 3;

    // per-thread description of the A rows it loads
    int a_base[A_CHUNKS], a_iy0[A_CHUNKS], a_ix0[A_CHUNKS];
    const int plane = p.ho * p.wo;
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
        const int m = m0 + lrow + i * ROWS_PER_PASS;
        if (m < p.m) {
            const int img = m / plane, r = m - img * plane;
            const int oy = r / p.wo, ox = r - oy * p.wo;
            a_iy0[i] = oy * p.stride_h + p.y_base;
            a_ix0[i] = ox * p.stride_w + p.x_base;
            a_base[i] = ((img * p.h + a_iy0[i]) * p.w + a_ix0[i]) * p.cin;
        } else {  // rows past M read nothing: every tap lands outside the image
            a_iy0[i] = -(1 << 20);
            a_ix0[i] = -(1 << 20);
            a_base[i] = 0;
        }
    }

    v16i acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    int rowsum[A_CHUNKS];
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) rowsum[i] = 0;
    const bool need_rowsum = p.zw != 0;

    const int k_tiles = p.k_pad / BK;
    uint4 ra[A_CHUNKS], rb[B_CHUNKS];

    auto load_stage = [&](int kt) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) ra[i] = load_a_chunk<VEC>(p, a_base[i], a_iy0[i], a_ix0[i], kt * 4 + kc);
#pragma unroll
        for (int i = 0; i < B_CHUNKS; ++i)
            rb[i] = *reinterpret_cast<const uint4 *>(p.b + (size_t)(n0 + lrow + i * ROWS_PER_PASS) * p.k_pad + kt * BK + kc * 16);
    };
    auto store_stage = [&](int buf) {
        uint8_t *as = lds + buf * STAGE_BYTES;
        uint8_t *bs = as + BM * LDS_ROW;
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            const uint4 v = xor128(ra[i], p.a_xor);
            if (need_rowsum) rowsum[i] = sum_bytes_signed(v, rowsum[i]);
            *reinterpret_cast<uint4 *>(as + (lrow + i * ROWS_PER_PASS) * LDS_ROW + kc * 16) = v;
        }
#pragma unroll
        for (int i = 0; i < B_CHUNKS; ++i)
            *reinterpret_cast<uint4 *>(bs + (lrow + i * ROWS_PER_PASS) * LDS_ROW + kc * 16) = rb[i];
    };

    load_stage(0);
    store_stage(0);
    __syncthreads();

    const int frag_row = lane & 31, frag_k = (lane >> 5) * 16;
    for (int kt = 0; kt < k_tiles; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < k_tiles) load_stage(kt + 1);
        const uint8_t *as = lds + buf * STAGE_BYTES + (wm * WTM + frag_row) * LDS_ROW + frag_k;
        const uint8_t *bs = lds + buf * STAGE_BYTES + BM * LDS_ROW + (wn * WTN + frag_row) * LDS_ROW + frag_k;
#pragma unroll
        for (int kk = 0; kk < BK / 32; ++kk) {
            v4i af[FM], bf[FN];
#pragma unroll
            for (int i = 0; i < FM; ++i) af[i] = *reinterpret_cast<const v4i *>(as + i * 32 * LDS_ROW + kk * 32);
#pragma unroll
            for (int j = 0; j < FN; ++j) bf[j] = *reinterpret_cast<const v4i *>(bs + j * 32 * LDS_ROW + kk * 32);
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < k_tiles) store_stage(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue: row sums -> LDS, requantize, stage the uint8 tile in LDS, coalesced store
    if (need_rowsum) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            int s = rowsum[i];
            s += __shfl_xor(s, 1);
            s += __shfl_xor(s, 2);
            if (kc == 0) rowsum_s[lrow + i * ROWS_PER_PASS] = s;
        }
    } else {
        for (int i = tid; i < BM; i += THREADS) rowsum_s[i] = 0;
    }
    __syncthreads();  // also: every wave is done reading the operand stages

    uint8_t *cs = lds;
    const RequantDev rq = p.rq;
#pragma unroll
    for (int j = 0; j < FN; ++j) {
        const int nl = wn * WTN + j * 32 + (lane & 31);
        const int32_t bias = p.bias[n0 + nl];
        const bool per_channel = rq.pc_multiplier != nullptr;
        const int32_t ch_mult = per_channel ? rq.pc_multiplier[n0 + nl] : 0, ch_shift = per_channel ? rq.pc_shift[n0 + nl] : 0;
#pragma unroll
        for (int i = 0; i < FM; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int ml = wm * WTM + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                const int32_t v = acc[i][j][r] + bias - p.zw * rowsum_s[ml];
                cs[ml * OUT_ROW + nl] =
                    (uint8_t)((per_channel ? requant_u8_channel(v, ch_mult, ch_shift, rq) : requant_u8(v, rq)) ^ (p.out_xor & 0xFFu));
            }
        }
    }
    __syncthreads();

    constexpr int CHUNKS_PER_ROW = BN / 16;
    const bool wide = (p.ldc & 15) == 0 && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
    for (int q = tid; q < BM * CHUNKS_PER_ROW; q += THREADS) {
        const int ml = q / CHUNKS_PER_ROW, nl = (q - ml * CHUNKS_PER_ROW) * 16;
        const int m = m0 + ml, n = n0 + nl;
        if (m >= p.m || n >= p.n) continue;
        const int img = m / plane, r = m - img * plane;
        const int oy = r / p.wo, ox = r - oy * p.wo;
        const size_t pix = ((size_t)img * p.out_h + (oy * p.out_sy + p.out_y0)) * p.out_w + (ox * p.out_sx + p.out_x0);
        uint8_t *dst = p.out + pix * p.ldc + n;
        const uint8_t *src = cs + ml * OUT_ROW + nl;
        if (wide && n + 16 <= p.n) {
            *reinterpret_cast<uint4 *>(dst) = *reinterpret_cast<const uint4 *>(src);
        } else {
            const uint4 v = *reinterpret_cast<const uint4 *>(src);
            const uint32_t packed[4] = {v.x, v.y, v.z, v.w};
            store_bytes_any_alignment(dst, packed, p.n - n < 16 ? p.n - n : 16);
        }
    }
}

template <int BM, int BN, int WGM, int WGN>
int launch_tile(const GemmProblem &p, hipStream_t stream) {
    const int tiles_m = (p.m + BM - 1) / BM, tiles_n = (p.n + BN - 1) / BN;
    const dim3 grid(tiles_m * tiles_n), block(WGM * WGN * 64);
    if (p.vec == 16)
        hipLaunchKernelGGL((igemm_u8_kernel<BM, BN, WGM, WGN, 16>), grid, block, 0, stream, p, tiles_m, tiles_n);
    else if (p.vec == 4)
        hipLaunchKernelGGL((igemm_u8_kernel<BM, BN, WGM, WGN, 4>), grid, block, 0, stream, p, tiles_m, tiles_n);
    else
        hipLaunchKernelGGL((igemm_u8_kernel<BM, BN, WGM, WGN, 1>), grid, block, 0, stream, p, tiles_m, tiles_n);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

}  // namespace

int igemm_n_tile(int32_t, int32_t, int32_t) { return 256; }

int launch_igemm(const GemmProblem &p, hipStream_t stream) {
    if (p.m <= 0 || p.n <= 0) return EH_OK;
    if (p.cfg.id == GEMM_THIN) return launch_igemm_thin(&p, 1, stream);
    if (p.cfg.id == GEMM_C3K3) return launch_conv_c3k3(p, stream);
    if (p.cfg.id == GEMM_CONV3X3) return launch_conv3x3_patch(p, stream);
    if (p.cfg.id == GEMM_ROWS) return launch_conv_rows(p, stream);
    if (p.cfg.id == GEMM_SKINNY) return launch_gemm_skinny(p, stream);
    EH_REQUIRE(p.k_pad % BK == 0 && p.k_pad > 0, "igemm: padded reduction length %d is not a multiple of %d", p.k_pad, BK);
    EH_REQUIRE(p.vec == 16 || p.vec == 4 || p.vec == 1, "igemm: bad load unit %d", p.vec);
    if (p.cfg.id != GEMM_STAGED) return launch_igemm_dma(&p, 1, stream);
    // Pick the largest tile that still spreads the problem over the 256 CUs.
    const long tiles128 = (long)((p.m + 127) / 128) * ((p.n + 127) / 128);
    const long tiles64 = (long)((p.m + 63) / 64) * ((p.n + 63) / 64);
    if (tiles128 >= 256 || tiles64 <= 64) {
        if (p.n > 64) return launch_tile<128, 128, 2, 2>(p, stream);
        return launch_tile<128, 64, 2, 2>(p, stream);
    }
    return launch_tile<64, 64, 2, 2>(p, stream);
}

int launch_igemm_batch(const GemmProblem *ps, int count, hipStream_t stream) {
    int i = 0;
    while (i < count) {
        const GemmProblem &p = ps[i];
        int run = 1;
        const bool dma = p.cfg.id != GEMM_STAGED && p.cfg.id != GEMM_THIN && p.cfg.id != GEMM_C3K3 && p.cfg.id != GEMM_CONV3X3 && p.cfg.id != GEMM_ROWS && p.cfg.id != GEMM_SKINNY && p.m > 0 && p.n > 0;
        if (dma)
            // (row counts may differ where nothing depends on them: table-driven problems; the launch covers the largest)
            while (i + run < count && run < GemmBatch::MAX && ps[i + run].cfg.id == p.cfg.id && (ps[i + run].m == p.m || (!p.dense && !p.partial)) &&
                   ps[i + run].n == p.n && ps[i + run].k_pad == p.k_pad && ps[i + run].dense == p.dense && ps[i + run].zw == p.zw)
                ++run;
        // ... and so do equally shaped one-tap problems (the phases of a transposed convolution whose kernel is its stride,
        // the groups of a grouped 1x1 convolution)
        const bool thin = p.cfg.id == GEMM_THIN && p.m > 0 && p.n > 0 && p.residual == nullptr;
        if (thin)
            while (i + run < count && run < GemmBatch::MAX && ps[i + run].cfg.id == GEMM_THIN && ps[i + run].residual == nullptr &&
                   ps[i + run].m == p.m && ps[i + run].n == p.n && ps[i + run].k == p.k && ps[i + run].k_pad == p.k_pad && ps[i + run].cin == p.cin &&
                   ps[i + run].ldc == p.ldc && ps[i + run].zw == p.zw && ps[i + run].ho == p.ho && ps[i + run].wo == p.wo && ps[i + run].h == p.h &&
                   ps[i + run].w == p.w && ps[i + run].stride_h == p.stride_h && ps[i + run].stride_w == p.stride_w && ps[i + run].out_sy == p.out_sy &&
                   ps[i + run].out_sx == p.out_sx && ps[i + run].out_h == p.out_h && ps[i + run].out_w == p.out_w &&
                   ps[i + run].y_base == p.y_base && ps[i + run].x_base == p.x_base &&
                   ps[i + run].rq.fast == p.rq.fast && (ps[i + run].rq.pc_multiplier != nullptr) == (p.rq.pc_multiplier != nullptr))
                ++run;
        int rc;
        if (thin && run > 1) {
            rc = launch_igemm_thin(ps + i, run, stream);
        } else if (dma && run > 1) {
            EH_REQUIRE(p.k_pad % 64 == 0 && p.k_pad > 0, "igemm: padded reduction length %d", p.k_pad);
            rc = launch_igemm_dma(ps + i, run, stream);
        } else {
            rc = launch_igemm(p, stream);
        }
        if (rc) return rc;
        i += run;
    }
    return EH_OK;
}

}  // namespace eh
