// Implicit-GEMM uint8 kernels for gfx950 whose operands go from HBM/L2 straight
// into LDS (global_load_lds_dwordx4), several reduction stages ahead of the
// matrix cores, with no register staging.  Used whenever the input channels come
// in 16-byte units; the register-staged kernel in eh_gemm.hip covers the rest.
//
// LDS image of one stage: rows of 64 reduction bytes, 16 rows per 1 KiB block,
// the four 16-byte chunks of a row XOR-swizzled by (row >> 1) & 3 so that the
// 32x32x32 MFMA fragment reads (32 rows x 16 bytes per half wave) are free of
// bank conflicts.  A wave-wide LDS-DMA instruction writes lane i at base + 16*i,
// so lane i fetches the global chunk that belongs in slot i: packed weights are
// stored in exactly this order (a linear 1 KiB copy per instruction), activation
// lanes compute their own addresses (implicit im2col), and lanes whose tap falls
// outside the image fetch from a 16-byte constant holding the input zero point.
//
// Activations stay uint8 in LDS; the -128 shift is one XOR per fragment register
// on the way to the MFMA, and the per-row activation sums needed when
// zp_w != 128 are v_dot4 accumulations over the same fragment registers.
#include "eh_internal.h"

namespace eh {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) uint8_t lds_byte;

namespace {

constexpr int BK = 64;
constexpr int16_t KPAD_MARK = INT16_MIN;

__device__ __forceinline__ uint32_t lds_offset(const void *p) {
    return (uint32_t)(uintptr_t)(lds_byte *)p;
}

// One wave copies 64 x 16 bytes: lane i's 16 bytes land at lds_base + 16 * i.
__device__ __forceinline__ void dma16(const void *gptr, uint32_t lds_base_uniform) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gptr), "s"(lds_base_uniform) : "memory");
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ v4i xor128(v4i v) {
    v.x ^= (int)0x80808080u;
    v.y ^= (int)0x80808080u;
    v.z ^= (int)0x80808080u;
    v.w ^= (int)0x80808080u;
    return v;
}

__device__ __forceinline__ int sum_bytes_signed(v4i v, int acc) {
    acc = __builtin_amdgcn_sdot4(v.x, 0x01010101, acc, false);
    acc = __builtin_amdgcn_sdot4(v.y, 0x01010101, acc, false);
    acc = __builtin_amdgcn_sdot4(v.z, 0x01010101, acc, false);
    acc = __builtin_amdgcn_sdot4(v.w, 0x01010101, acc, false);
    return acc;
}

// Where one activation row (one output pixel) starts in the input image.
struct RowRef {
    int base;  // byte offset of the top-left tap (may be negative: the tap may lie in the padding)
    int iy0, ix0;
};

__device__ __forceinline__ RowRef make_row(const GemmProblem &p, int m, int plane) {
    RowRef r;
    if (m < p.m) {
        const int img = m / plane, rem = m - img * plane;
        const int oy = rem / p.wo, ox = rem - oy * p.wo;
        r.iy0 = oy * p.stride_h + p.y_base;
        r.ix0 = ox * p.stride_w + p.x_base;
        r.base = ((img * p.h + r.iy0) * p.w + r.ix0) * p.cin;
    } else {  // rows past M: every tap is "outside", they read the constant
        r.iy0 = -(1 << 20);
        r.ix0 = -(1 << 20);
        r.base = 0;
    }
    return r;
}

__device__ __forceinline__ const uint8_t *a_chunk_address(const GemmProblem &p, const RowRef &r, const KUnit ku) {
    const int iy = r.iy0 + ku.dy, ix = r.ix0 + ku.dx;
    if (ku.dy == KPAD_MARK) return p.fillbuf + 16;  // reduction padding: 0x80 bytes, i.e. zero after the shift
    if ((unsigned)iy < (unsigned)p.h && (unsigned)ix < (unsigned)p.w) return p.a + (r.base + ku.offset);
    return p.fillbuf;  // spatial padding: the input zero point
}

__device__ __forceinline__ int frag_offset(int row, int chunk) { return row * 64 + ((chunk ^ ((row >> 1) & 3)) << 4); }

// ---------------------------------------------------------------------------
// Cooperative kernel: 2 x 2 waves share a BM x BN tile; one barrier per stage.
// ---------------------------------------------------------------------------
template <int BM, int BN, int STAGES>
__global__ __launch_bounds__(256) void igemm_dma_tile_kernel(const GemmProblem p, const int tiles_m, const int tiles_n) {
    constexpr int WTM = BM / 2, WTN = BN / 2;
    constexpr int FM = WTM / 32, FN = WTN / 32;
    constexpr int A_LOADS = BM / 64, B_LOADS = BN / 64;  // wave-wide DMA instructions per wave per stage
    constexpr int LPS = A_LOADS + B_LOADS;
    constexpr int STAGE_BYTES = (BM + BN) * BK;
    constexpr int OUT_ROW = BN + 16;
    static_assert(BM % 64 == 0 && BN % 64 == 0, "tile extents are multiples of 64");
    static_assert((STAGES - 2) * LPS <= 63, "vmcnt is a 6-bit counter");
    static_assert(BM * OUT_ROW <= STAGES * STAGE_BYTES, "output staging reuses the operand stages");

    __shared__ __align__(1024) uint8_t stages[STAGES * STAGE_BYTES];
    __shared__ int32_t rowsum_s[BM];
    extern __shared__ __align__(8) uint8_t ktab_s_raw[];
    KUnit *ktab_s = reinterpret_cast<KUnit *>(ktab_s_raw);

    int tile = blockIdx.x;
    const int total = tiles_m * tiles_n;
    if ((total & 7) == 0) tile = (blockIdx.x & 7) * (total >> 3) + (blockIdx.x >> 3);
    const int tm = tile % tiles_m, tn = tile / tiles_m;
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 1, wn = wave >> 1;
    const int k_tiles = p.k_pad / BK;

    for (int i = tid; i < k_tiles * 4; i += 256) ktab_s[i] = p.ktab[i];

    // this lane's slot in a DMA block: row (lane >> 2) of 16, physical chunk lane & 3
    const int slot_row = lane >> 2;
    const int my_chunk = (lane & 3) ^ ((slot_row >> 1) & 3);
    const int plane = p.ho * p.wo;
    RowRef rows[A_LOADS];
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) rows[i] = make_row(p, m0 + (i * 4 + wave) * 16 + slot_row, plane);
    const int8_t *b_src = p.b + ((size_t)(n0 >> 4) * k_tiles) * 1024 + lane * 16;
    const uint32_t lds0 = lds_offset(stages);
    __syncthreads();

    auto issue = [&](int kt) {
        const uint32_t sbase = lds0 + (kt % STAGES) * STAGE_BYTES;
        const KUnit ku = ktab_s[kt * 4 + my_chunk];
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i)
            dma16(a_chunk_address(p, rows[i], ku), sbase + ((i * 4 + wave) << 10));
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i) {
            const int blk = i * 4 + wave;
            dma16(b_src + ((size_t)blk * k_tiles + kt) * 1024, sbase + BM * BK + (blk << 10));
        }
    };

    v16i acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
    int rowsum[FM];
#pragma unroll
    for (int i = 0; i < FM; ++i) rowsum[i] = 0;
    const bool need_rowsum = p.zw != 0 && wn == 0;

#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
        if (s < k_tiles) issue(s);

    const int frow = lane & 31, fhalf = lane >> 5;
    for (int kt = 0; kt < k_tiles; ++kt) {
        // loads of the stages after kt may stay in flight; in the tail just drain
        if (k_tiles - 1 - kt >= STAGES - 2)
            wait_vmcnt<(STAGES - 2) * LPS>();
        else
            wait_vmcnt<0>();
        __syncthreads();
        if (kt + STAGES - 1 < k_tiles) issue(kt + STAGES - 1);
        const uint8_t *as = stages + (kt % STAGES) * STAGE_BYTES;
        const uint8_t *bs = as + BM * BK;
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            v4i af[FM], bf[FN];
#pragma unroll
            for (int i = 0; i < FM; ++i) {
                const int row = wm * WTM + i * 32 + frow;
                af[i] = xor128(*reinterpret_cast<const v4i *>(as + frag_offset(row, kk * 2 + fhalf)));
                if (need_rowsum) rowsum[i] = sum_bytes_signed(af[i], rowsum[i]);
            }
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                const int row = wn * WTN + j * 32 + frow;
                bf[j] = *reinterpret_cast<const v4i *>(bs + frag_offset(row, kk * 2 + fhalf));
            }
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
    }

    // ---- epilogue
    if (p.zw != 0) {
        if (wn == 0) {
#pragma unroll
            for (int i = 0; i < FM; ++i) {
                const int s = rowsum[i] + __shfl_xor(rowsum[i], 32);
                if (fhalf == 0) rowsum_s[wm * WTM + i * 32 + frow] = s;
            }
        }
    } else {
        for (int i = tid; i < BM; i += 256) rowsum_s[i] = 0;
    }
    __syncthreads();  // row sums visible; every wave is done with the operand stages

    uint8_t *cs = stages;
    const RequantDev rq = p.rq;
#pragma unroll
    for (int j = 0; j < FN; ++j) {
        const int nl = wn * WTN + j * 32 + frow;
        const int32_t bias = p.bias[n0 + nl];
#pragma unroll
        for (int i = 0; i < FM; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int ml = wm * WTM + i * 32 + 8 * (r >> 2) + 4 * fhalf + (r & 3);
                const int32_t v = acc[i][j][r] + bias - p.zw * rowsum_s[ml];
                cs[ml * OUT_ROW + nl] = (uint8_t)requant_u8(v, rq);
            }
        }
    }
    __syncthreads();

    constexpr int CHUNKS_PER_ROW = BN / 16;
    const bool wide = (p.ldc & 15) == 0 && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
    for (int q = tid; q < BM * CHUNKS_PER_ROW; q += 256) {
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
            const int cnt = p.n - n < 16 ? p.n - n : 16;
            for (int t = 0; t < cnt; ++t) dst[t] = src[t];
        }
    }
}

// ---------------------------------------------------------------------------
// Split-reduction kernel for problems with few output tiles: the four waves of a
// workgroup share one 64 x 64 output tile and each takes every fourth 64-byte
// slice of the reduction axis through its own private LDS ring, so the main loop
// has no barrier at all; the four partial tiles meet in LDS at the end.
// ---------------------------------------------------------------------------
template <int STAGES>
__global__ __launch_bounds__(256) void igemm_dma_splitk_kernel(const GemmProblem p, const int tiles_m, const int tiles_n) {
    constexpr int BM = 64, BN = 64, FM = 2, FN = 2;
    constexpr int LPS = 8;  // 4 activation + 4 weight DMA instructions per stage
    constexpr int STAGE_BYTES = (BM + BN) * BK;
    constexpr int RING_BYTES = STAGES * STAGE_BYTES;
    constexpr int PART_ROW = BN + 4;  // int32 elements per row of a partial tile
    static_assert((STAGES - 2) * LPS <= 63, "vmcnt is a 6-bit counter");
    static_assert(4 * RING_BYTES >= 4 * BM * PART_ROW * 4, "partial tiles reuse the rings");

    __shared__ __align__(1024) uint8_t rings[4 * RING_BYTES];
    __shared__ int32_t rowsum_s[8][BM];
    extern __shared__ __align__(8) uint8_t ktab_s_raw[];
    KUnit *ktab_s = reinterpret_cast<KUnit *>(ktab_s_raw);

    int tile = blockIdx.x;
    const int total = tiles_m * tiles_n;
    if ((total & 7) == 0) tile = (blockIdx.x & 7) * (total >> 3) + (blockIdx.x >> 3);
    const int tm = tile % tiles_m, tn = tile / tiles_m;
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int k_tiles = p.k_pad / BK;
    for (int i = tid; i < k_tiles * 4; i += 256) ktab_s[i] = p.ktab[i];

    const int slot_row = lane >> 2;
    const int my_chunk = (lane & 3) ^ ((slot_row >> 1) & 3);
    const int plane = p.ho * p.wo;
    RowRef rows[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) rows[i] = make_row(p, m0 + i * 16 + slot_row, plane);
    const int8_t *b_src = p.b + ((size_t)(n0 >> 4) * k_tiles) * 1024 + lane * 16;
    uint8_t *ring = rings + wave * RING_BYTES;
    const uint32_t lds0 = lds_offset(ring);
    __syncthreads();

    // this wave's slices: kt = wave, wave + 4, ...
    const int my_tiles = (k_tiles - wave + 3) >> 2;
    auto issue = [&](int it) {
        const int kt = wave + (it << 2);
        const uint32_t sbase = lds0 + (it % STAGES) * STAGE_BYTES;
        const KUnit ku = ktab_s[kt * 4 + my_chunk];
#pragma unroll
        for (int i = 0; i < 4; ++i) dma16(a_chunk_address(p, rows[i], ku), sbase + (i << 10));
#pragma unroll
        for (int i = 0; i < 4; ++i) dma16(b_src + ((size_t)i * k_tiles + kt) * 1024, sbase + BM * BK + (i << 10));
    };

    v16i acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
    int rowsum[FM] = {0, 0};
    const bool need_rowsum = p.zw != 0;

#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
        if (s < my_tiles) issue(s);

    const int frow = lane & 31, fhalf = lane >> 5;
    for (int it = 0; it < my_tiles; ++it) {
        if (my_tiles - 1 - it >= STAGES - 2)
            wait_vmcnt<(STAGES - 2) * LPS>();
        else
            wait_vmcnt<0>();
        // The stage refilled below was read in the previous iteration by this same
        // wave; its LDS reads have returned (their values fed the MFMAs already issued).
        if (it + STAGES - 1 < my_tiles) issue(it + STAGES - 1);
        const uint8_t *as = ring + (it % STAGES) * STAGE_BYTES;
        const uint8_t *bs = as + BM * BK;
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            v4i af[FM], bf[FN];
#pragma unroll
            for (int i = 0; i < FM; ++i) {
                af[i] = xor128(*reinterpret_cast<const v4i *>(as + frag_offset(i * 32 + frow, kk * 2 + fhalf)));
                if (need_rowsum) rowsum[i] = sum_bytes_signed(af[i], rowsum[i]);
            }
#pragma unroll
            for (int j = 0; j < FN; ++j) bf[j] = *reinterpret_cast<const v4i *>(bs + frag_offset(j * 32 + frow, kk * 2 + fhalf));
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
    }

    // ---- meet in LDS
    __syncthreads();  // every wave has finished reading its ring
    int32_t *part = reinterpret_cast<int32_t *>(rings) + wave * BM * PART_ROW;
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int ml = i * 32 + 8 * (r >> 2) + 4 * fhalf + (r & 3);
                part[ml * PART_ROW + j * 32 + frow] = acc[i][j][r];
            }
#pragma unroll
    for (int i = 0; i < FM; ++i) rowsum_s[wave * 2 + fhalf][i * 32 + frow] = rowsum[i];
    __syncthreads();

    // thread -> row tid / 4, sixteen columns starting at (tid & 3) * 16
    const int ml = tid >> 2, nl = (tid & 3) * 16;
    const int m = m0 + ml, n = n0 + nl;
    if (m >= p.m || n >= p.n) return;
    int rs = 0;
    if (need_rowsum) {
#pragma unroll
        for (int w = 0; w < 8; ++w) rs += rowsum_s[w][ml];
    }
    const int32_t *pr = reinterpret_cast<const int32_t *>(rings) + ml * PART_ROW + nl;
    const RequantDev rq = p.rq;
    uint32_t packed[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const int4 s0 = *reinterpret_cast<const int4 *>(pr + g * 4);
        const int4 s1 = *reinterpret_cast<const int4 *>(pr + g * 4 + BM * PART_ROW);
        const int4 s2 = *reinterpret_cast<const int4 *>(pr + g * 4 + 2 * BM * PART_ROW);
        const int4 s3 = *reinterpret_cast<const int4 *>(pr + g * 4 + 3 * BM * PART_ROW);
        const int4 bb = *reinterpret_cast<const int4 *>(p.bias + n + g * 4);
        const int corr = p.zw * rs;
        const uint32_t o0 = requant_u8(s0.x + s1.x + s2.x + s3.x + bb.x - corr, rq);
        const uint32_t o1 = requant_u8(s0.y + s1.y + s2.y + s3.y + bb.y - corr, rq);
        const uint32_t o2 = requant_u8(s0.z + s1.z + s2.z + s3.z + bb.z - corr, rq);
        const uint32_t o3 = requant_u8(s0.w + s1.w + s2.w + s3.w + bb.w - corr, rq);
        packed[g] = o0 | (o1 << 8) | (o2 << 16) | (o3 << 24);
    }
    const int img = m / plane, r = m - img * plane;
    const int oy = r / p.wo, ox = r - oy * p.wo;
    const size_t pix = ((size_t)img * p.out_h + (oy * p.out_sy + p.out_y0)) * p.out_w + (ox * p.out_sx + p.out_x0);
    uint8_t *dst = p.out + pix * p.ldc + n;
    const bool wide = (p.ldc & 15) == 0 && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
    if (wide && n + 16 <= p.n) {
        *reinterpret_cast<uint4 *>(dst) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
    } else {
        const int cnt = p.n - n < 16 ? p.n - n : 16;
        for (int t = 0; t < cnt; ++t) dst[t] = (uint8_t)(packed[t >> 2] >> (8 * (t & 3)));
    }
}

template <int BM, int BN, int STAGES>
int launch_tile(const GemmProblem &p, hipStream_t stream) {
    const int tiles_m = (p.m + BM - 1) / BM, tiles_n = (p.n + BN - 1) / BN;
    const size_t ktab_bytes = (size_t)(p.k_pad / 16) * sizeof(KUnit);
    hipLaunchKernelGGL((igemm_dma_tile_kernel<BM, BN, STAGES>), dim3(tiles_m * tiles_n), dim3(256), ktab_bytes, stream, p,
                       tiles_m, tiles_n);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

}  // namespace

size_t igemm_dma_ktab_limit() { return 16384; }

int launch_igemm_dma(const GemmProblem &p, hipStream_t stream) {
    const size_t ktab_bytes = (size_t)(p.k_pad / 16) * sizeof(KUnit);
    EH_REQUIRE(p.vec == 16 && ktab_bytes <= igemm_dma_ktab_limit(), "igemm_dma: unsupported problem");
    const long t256 = (long)((p.m + 255) / 256) * ((p.n + 127) / 128);
    const long t128 = (long)((p.m + 127) / 128) * ((p.n + 127) / 128);
    if (p.n > 64 && t256 >= 256) return launch_tile<256, 128, 3>(p, stream);
    if (p.n > 64 && t128 >= 192) return launch_tile<128, 128, 3>(p, stream);
    const int tiles_m = (p.m + 63) / 64, tiles_n = (p.n + 63) / 64;
    hipLaunchKernelGGL((igemm_dma_splitk_kernel<4>), dim3(tiles_m * tiles_n), dim3(256), ktab_bytes, stream, p, tiles_m,
                       tiles_n);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

}  // namespace eh
