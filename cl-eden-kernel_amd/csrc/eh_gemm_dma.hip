// Implicit-GEMM uint8 kernel for gfx950 whose operands go from HBM/L2 straight
// into LDS (global_load_lds_dwordx4), several reduction stages ahead of the
// matrix cores, with no register staging.  Used whenever the input channels come
// in 16-byte units; the register-staged kernel in eh_gemm.hip covers the rest.
//
// One stage holds a SLAB-byte slice of the reduction axis (128 or 256 bytes, so
// every activation row is fetched in whole 128-byte cache lines) for BM
// activation rows and BN weight rows.  LDS rows are SLAB bytes; the 16-byte
// chunks of a row are XOR-swizzled by the row index so that the 32x32x32 MFMA
// fragment reads (32 rows x 16 bytes per half wave) are free of bank conflicts.
// A wave-wide LDS-DMA instruction writes lane i at base + 16*i, so lane i
// fetches the global chunk that belongs in slot i: packed weights are stored in
// exactly this order (a linear 1 KiB copy per instruction), activation lanes
// compute their own addresses (implicit im2col), and lanes whose tap falls
// outside the image fetch a 16-byte constant holding the input zero point.
//
// The 4 waves of a workgroup are arranged WGM x WGN x WGK.  WGK > 1 splits the
// slab along the reduction axis between waves (each wave still owns the whole
// BM/WGM x BN/WGN sub-tile): for problems with few output tiles this keeps LDS
// traffic per MFMA low; the partial tiles meet in LDS at the end (exact: int32).
//
// The MFMA is issued with the weight fragment as its row operand and the packed
// weight rows of every 32-channel block are permuted, so a lane ends up holding,
// for ONE output pixel, sixteen consecutive output channels: sixteen requantized
// bytes go out in one 16-byte store to the channels-last output with no LDS round
// trip, and the per-pixel terms are per-lane scalars.
//
// Activations stay uint8 in LDS; the -128 shift is one XOR per fragment register
// on the way to the MFMA, and the per-row activation sums needed when
// zp_w != 128 are v_dot4 accumulations over the same fragment registers.
#include <type_traits>
#include <utility>

#include "eh_internal.h"

namespace eh {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) uint8_t lds_byte;

namespace {

constexpr int16_t KPAD_MARK = INT16_MIN;

__device__ __forceinline__ uint32_t lds_offset(const void *p) { return (uint32_t)(uintptr_t)(lds_byte *)p; }

// One wave copies 64 x 16 bytes: lane i's 16 bytes land at lds_base + 16 * i.
__device__ __forceinline__ void dma16(const void *gptr, uint32_t lds_base_uniform) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gptr), "s"(lds_base_uniform) : "memory");
}

// The same with the address split into a wave-uniform base and a 32-bit per-lane offset.
__device__ __forceinline__ void dma16_off(const void *base_uniform, uint32_t lane_offset, uint32_t lds_base_uniform) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_offset), "s"(base_uniform),
                 "s"(lds_base_uniform)
                 : "memory");
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ v4i xor128(v4i v, int x) {
    v.x ^= x;
    v.y ^= x;
    v.z ^= x;
    v.w ^= x;
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
    int yx;    // (iy0 << 16) | (ix0 & 0xFFFF), both signed 16-bit
};

__device__ __forceinline__ RowRef make_row(const GemmProblem &p, int m, int plane) {
    RowRef r;
    if (m < p.m) {
        const int img = (int)fastdiv((uint32_t)m, p.div_plane), rem = m - img * plane;
        const int oy = (int)fastdiv((uint32_t)rem, p.div_wo), ox = rem - oy * p.wo;
        const int iy0 = oy * p.stride_h + p.y_base, ix0 = ox * p.stride_w + p.x_base;
        r.base = ((img * p.h + iy0) * p.w + ix0) * p.cin;
        r.yx = (int)(((uint32_t)iy0 << 16) | ((uint32_t)ix0 & 0xFFFFu));
    } else {  // rows past M: every tap is "outside", they read the constant
        r.base = 0;
        r.yx = (int)0x80008000u;
    }
    return r;
}

__device__ __forceinline__ const uint8_t *a_chunk_address(const GemmProblem &p, const RowRef &r, const KUnit ku) {
    const int iy = (r.yx >> 16) + ku.dy, ix = (int)(short)(r.yx & 0xFFFF) + ku.dx;
    const bool inside = (unsigned)iy < (unsigned)p.h && (unsigned)ix < (unsigned)p.w;
    // reduction padding reads 0x80 bytes (zero after the shift); spatial padding reads the input zero point
    const uintptr_t image = reinterpret_cast<uintptr_t>(p.a) + (intptr_t)(r.base + ku.offset);
    const uintptr_t constant = reinterpret_cast<uintptr_t>(p.fillbuf) + (ku.dy == KPAD_MARK ? 16 : 0);
    return reinterpret_cast<const uint8_t *>(inside && ku.dy != KPAD_MARK ? image : constant);
}

// byte offset of output pixel m (row of the GEMM) in the channels-last output
__device__ __forceinline__ size_t out_pixel_offset(const GemmProblem &p, int m, int plane) {
    const int img = (int)fastdiv((uint32_t)m, p.div_plane), rem = m - img * plane;
    const int oy = (int)fastdiv((uint32_t)rem, p.div_wo), ox = rem - oy * p.wo;
    return (((size_t)img * p.out_h + (oy * p.out_sy + p.out_y0)) * p.out_w + (ox * p.out_sx + p.out_x0)) * (size_t)p.ldc;
}

template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F &&f) {
    (f(std::integral_constant<int, I>{}), ...);
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>), unrolled at compile time
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

// DENSE: 0 table-driven operand gather; 1 a plain matrix of whole slabs; 2 a plain matrix whose reduction ends inside
// its last slab (the chunks past the end read a constant that the sign flip turns into 0).
template <int BM, int BN, int WGM, int WGN, int WGK, int SLAB, int STAGES, int DENSE, bool ROWSUM>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(BM == 128 && BN == 64 ? 3 : (BM == 128 && BN == 128 ? 2 : 1)))) void igemm_dma_kernel(const GemmBatch batch, const int count, const int tiles_m, const int tiles_n,
                                                        const int gm, const int gn) {
    static_assert(WGM * WGN * WGK == 4, "four waves per workgroup");
    constexpr int CPR = SLAB / 16;            // 16-byte chunks per LDS row
    constexpr int RPB = 1024 / SLAB;          // rows per 1 KiB DMA block
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int FM = WTM / 32, FN = WTN / 32;
    constexpr int KSTEPS = SLAB / WGK / 32;   // 32-byte MFMA steps per wave per stage
    constexpr int A_LOADS = BM / RPB / 4, B_LOADS = BN / RPB / 4;  // DMA instructions per wave per stage
    constexpr int LPS = A_LOADS + B_LOADS;
    constexpr int STAGE_BYTES = (BM + BN) * SLAB;
    constexpr int PART_ROW = BN + 4;          // int32 per row of a partial tile: 8 consecutive rows cover all banks
    constexpr int NMF = FM * FN;              // MFMAs per step
    constexpr int NREADS = FM + FN;           // fragment reads per step
    constexpr int RPS = (NREADS + NMF - 1) / NMF;                    // fragment reads placed behind one MFMA
    constexpr int WINDOW = STAGES == 2 ? KSTEPS / 2 : KSTEPS;        // steps over which the DMA of one stage is issued
    constexpr int DPS = (LPS + WINDOW * NMF - 1) / (WINDOW * NMF);   // DMA instructions placed behind one MFMA
    static_assert(WTM % 32 == 0 && WTN % 32 == 0 && KSTEPS >= 2 && KSTEPS % 2 == 0, "wave tile is made of 32x32x32 MFMA steps; fragment registers alternate between two sets");
    static_assert(BM % (RPB * 4) == 0 && BN % (RPB * 4) == 0, "whole DMA blocks per wave");
    static_assert((STAGES - 1) * LPS <= 63, "vmcnt is a 6-bit counter");
    // the WGK partial tiles of the split reduction reuse the operand stages; with two stages they need a little more
    constexpr int PARTIAL_BYTES = WGK == 1 ? 0 : WGK * BM * PART_ROW * 4;
    constexpr int STAGE_AREA = STAGES * STAGE_BYTES > PARTIAL_BYTES ? STAGES * STAGE_BYTES : PARTIAL_BYTES;
    static_assert(WGK == 1 || (BM == 64 && BN == 64 && WGM == 1 && WGN == 1), "the split-reduction epilogue is written for one 64x64 tile");
    static_assert(WTM % CPR == 0 && WTN % CPR == 0, "every fragment row of a lane has the same swizzle");

    __shared__ __align__(1024) uint8_t stages[STAGE_AREA];
    __shared__ int32_t rowsum_s[WGK * 2][BM];
    __shared__ __align__(16) int32_t bias_s[BN];  // read in the epilogue from LDS: a global load there would have to
                                                   // wait for the stores issued before it (one counter for both)
    // fused residual add (split-reduction epilogue only): the rescaled value of every possible residual byte and of
    // every possible result byte, so that an output costs two lookups and one rescaling instead of three rescalings
    __shared__ int32_t add_lut_s[WGK == 1 ? 1 : 2][WGK == 1 ? 1 : 256];
    extern __shared__ __align__(8) uint8_t ktab_s_raw[];
    KUnit *ktab_s = reinterpret_cast<KUnit *>(ktab_s_raw);

    // Workgroups are dispatched round-robin over the 8 XCDs, each with its own L2, and an
    // XCD runs up to 32 of these workgroups at a time (one per CU).  Tiles are therefore
    // handed out in groups that form a gm x gn rectangle of the output (32 tiles, fewer when
    // the whole launch has too few tiles to give every XCD a group): the workgroups of a
    // group walk the reduction axis in step, so every activation slab is pulled into that
    // L2 once for gn tiles and every weight slab once for gm tiles.  Equally shaped
    // problems of one operator (convolution groups, deconvolution phases) share a launch:
    // their groups are numbered one problem after the other.
    // Rectangles leave slots empty where they overhang the tile grid.  A launch with few tiles cannot afford that (the
    // empty slots push real tiles into a second round of workgroups): gm == 0 selects a plain split instead, every XCD
    // taking gn consecutive tiles of the problems' tiles in row-major order (neighbours share their activation rows).
    const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
    int which, tm, tn;
    if (gm == 0) {
        const int t_all = xcd * gn + j;
        const int per_problem = tiles_m * tiles_n;
        which = __builtin_amdgcn_readfirstlane(t_all / per_problem);
        const int t = t_all - which * per_problem;
        tm = __builtin_amdgcn_readfirstlane(t / tiles_n);
        tn = t - tm * tiles_n;
        if (which >= count) return;
    } else {
        const int gs = gm * gn;
        const int jg = __builtin_amdgcn_readfirstlane(j / gs);
        const int group_all = jg * 8 + xcd, within = j - jg * gs;
        const int groups_m = (tiles_m + gm - 1) / gm, groups_n = (tiles_n + gn - 1) / gn;
        // (the divisions run on the vector unit: tell the compiler their results are wave-uniform)
        which = __builtin_amdgcn_readfirstlane(group_all / (groups_m * groups_n));
        const int group = group_all - which * (groups_m * groups_n);
        if (which >= count) return;
        const int gj = __builtin_amdgcn_readfirstlane(group / groups_m), gi = group - gj * groups_m;
        const int wj = __builtin_amdgcn_readfirstlane(within / gm), wi = within - wj * gm;
        tm = gi * gm + wi;
        tn = gj * gn + wj;
        if (tm >= tiles_m || tn >= tiles_n) return;
    }
    const GemmProblem &p = batch.p[which];
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x, lane = tid & 63;
    // issued first and consumed after the main loop: by then it has long arrived
    static_assert(BN <= 256, "one bias value per thread");
    const int32_t bias_reg = tid < BN ? p.bias[n0 + tid] : 0;
    if constexpr (WGK != 1) {
        if (p.residual) {  // 256 threads, 256 byte values; visible after the barriers that precede the epilogue
            add_lut_s[0][tid] = mul_round_shift((int32_t)((uint32_t)(tid - p.radd.zp_a) << p.radd.left_shift), p.radd.mult_a, p.radd.rs_a);
            add_lut_s[1][tid] = mul_round_shift((int32_t)((uint32_t)(tid - p.radd.zp_b) << p.radd.left_shift), p.radd.mult_b, p.radd.rs_b);
        }
    }
    // the sixteen residual bytes this thread's outputs will be added to travel under the whole main loop as well
    uint4 res_reg = make_uint4(0, 0, 0, 0);
    bool res_vec = false;
    if constexpr (WGK != 1) {
        if (p.residual) {
            const int m = m0 + (tid & 63), n = n0 + (tid >> 6) * 16;
            res_vec = m < p.m && n + 16 <= p.n && (p.ldc & 15) == 0 && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0) &&
                      (reinterpret_cast<uintptr_t>(p.residual) & 15) == 0;
            if (res_vec) res_reg = *reinterpret_cast<const uint4 *>(p.residual + out_pixel_offset(p, m, p.ho * p.wo) + n);
        }
    }
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WGM, wn = (wave / WGM) % WGN, wk = wave / (WGM * WGN);
    const int k_slabs = p.k_pad / SLAB;
    const int a_xor = (int)p.a_xor;  // stored activation bytes -> int8 operands (uniform)

    // ---- operand fetch.  This lane's slot in a DMA block: row (lane / CPR), physical chunk lane % CPR.
    const int slot_row = lane / CPR;
    const int my_chunk = (lane % CPR) ^ ((wave * RPB + slot_row) & (CPR - 1));
    const int plane = p.ho * p.wo;
    RowRef rows[DENSE ? 1 : A_LOADS];
    uint32_t a_voff[DENSE ? A_LOADS : 1];  // dense: where this lane's chunk sits in the activation matrix, per DMA block
    const uint8_t *a_base = p.a;           // dense: uniform, advances by one slab per issued stage
    if constexpr (DENSE) {
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) {
            int m = m0 + (i * 4 + wave) * RPB + slot_row;
            m = m < p.m ? m : p.m - 1;  // rows past M re-read the last row; their results are never stored
            a_voff[i] = (uint32_t)m * (uint32_t)p.cin + my_chunk * 16;
        }
    } else {
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) rows[i] = make_row(p, m0 + (i * 4 + wave) * RPB + slot_row, plane);
    }
    // dense operands whose reduction is not whole slabs: which lanes' chunks lie past its end in the last slab
    constexpr bool ragged = DENSE == 2;
    const bool tail_lane = ragged && my_chunk * 16 >= p.k - (k_slabs - 1) * SLAB;
    auto tail_unit = [&](int slab) {
        KUnit ku = KUnit();
        ku.dy = (int16_t)(ragged && slab == k_slabs - 1 ? 1 : 0);
        return ku;
    };
    const int8_t *b_base[B_LOADS];  // uniform: the packed 1 KiB blocks of this wave's weight rows, slab 0
    // (only the split-reduction tile runs slices of a reduction, whose row blocks lie a whole reduction apart)
    const int b_block_slabs = (WGK != 1 && p.b_slabs) ? p.b_slabs : k_slabs;
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) b_base[i] = p.b + ((size_t)(n0 / RPB + i * 4 + wave) * b_block_slabs) * 1024;
    uint32_t b_voff = lane * 16;    // advances by one block per issued stage
    const uint32_t wave_lds = lds_offset(stages) + (wave << 10);

    auto issue_piece = [&](auto idx_c, const uint32_t stage_off, const KUnit ku) {
        constexpr int idx = decltype(idx_c)::value;
        if constexpr (idx < A_LOADS) {
            const uint32_t dst = wave_lds + stage_off + idx * 4096;
            if constexpr (DENSE) {
                // (ku.dy marks the last slab of a reduction that ends inside it: the chunks past its end read the
                // constant that the sign flip turns into 0 instead of the next pixel's bytes)
                if (DENSE == 1 || ku.dy == 0)
                    dma16_off(a_base, a_voff[idx], dst);
                else
                    dma16(tail_lane ? p.fillbuf + 16 : a_base + a_voff[idx], dst);
            } else
                dma16(a_chunk_address(p, rows[idx], ku), dst);
        } else {
            constexpr int bi = idx - A_LOADS;
            dma16_off(b_base[bi], b_voff, wave_lds + stage_off + BM * SLAB + bi * 4096);
        }
    };
    auto advance_slab = [&]() {
        if constexpr (DENSE) a_base += SLAB;
        b_voff += 1024;
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

    // ---- prologue: every stage buffer is filled.  The table-driven path sends the weight
    // blocks of the first stage ahead, so the copy of the k-table to LDS runs under their latency.
    if constexpr (!DENSE) {
        static_for<B_LOADS>([&](auto bi) { issue_piece(std::integral_constant<int, A_LOADS + decltype(bi)::value>{}, 0u, KUnit()); });
        for (int i = tid; i < k_slabs * CPR; i += 256) ktab_s[i] = p.ktab[i];
        __syncthreads();
        const KUnit ku = ktab_s[my_chunk];
        static_for<A_LOADS>([&](auto ai) { issue_piece(ai, 0u, ku); });
        advance_slab();
    }
#pragma unroll
    for (int s = DENSE ? 0 : 1; s < STAGES; ++s) {
        if (s < k_slabs) {
            KUnit ku = tail_unit(s);
            if constexpr (!DENSE) ku = ktab_s[s * CPR + my_chunk];
            static_for<LPS>([&](auto idx) { issue_piece(idx, (uint32_t)(s * STAGE_BYTES), ku); });
            advance_slab();
        }
    }

    // ---- main loop.  A SIMD runs one wave here and issues its instructions in order, one
    // per four clocks, while an MFMA occupies the matrix pipe for 32: the pipe stays busy only
    // if the other work of a step (fragment reads for the following step, the DMA of a later
    // stage, the signed shift of the activation fragments) is issued in the shadow of the
    // MFMAs, a few instructions behind each one.  The order below is written out slot by slot
    // and fenced, because the compiler otherwise gathers the MFMAs of a step into one block.
    //
    // Fragment registers alternate between two sets, so a stage buffer has been read completely
    // one step before its MFMAs end.  In the last step of slab s every wave waits for its own
    // DMA of slab s+1 and meets the others at a barrier; behind that barrier slab s+1 is visible
    // to all and the buffer of slab s is free, so the DMA of slab s+STAGES is issued into it
    // from that step on.
    const int frow = lane & 31, fhalf = lane >> 5;
    v4i af[2][FM], bf[2][FN];
    // read number r of a step, in order of first use: A0, B0 .. B(FN-1), A1 .. A(FM-1)
    auto read_frag = [&](auto r_c, auto buf_c, const uint8_t *stage, const int chunk_base) {
        constexpr int r = decltype(r_c)::value, buf = decltype(buf_c)::value;
        const int chunk = wk * (CPR / WGK) + chunk_base + fhalf;
        if constexpr (r == 0 || r > FN) {
            constexpr int i = r == 0 ? 0 : r - FN;
            const int row = wm * WTM + i * 32 + frow;
            af[buf][i] = *reinterpret_cast<const v4i *>(stage + row * SLAB + ((chunk ^ (row & (CPR - 1))) << 4));
        } else {
            constexpr int jj = r - 1;
            const int row = wn * WTN + jj * 32 + frow;
            bf[buf][jj] = *reinterpret_cast<const v4i *>(stage + BM * SLAB + row * SLAB + ((chunk ^ (row & (CPR - 1))) << 4));
        }
    };
    auto flip = [&](auto buf_c, auto i_c) {
        constexpr int buf = decltype(buf_c)::value, i = decltype(i_c)::value;
        af[buf][i] = xor128(af[buf][i], a_xor);
        if constexpr (ROWSUM) rowsum[i] = sum_bytes_signed(af[buf][i], rowsum[i]);
    };
    typedef std::integral_constant<int, 0> c0;
    typedef std::integral_constant<int, -1> no_wait;

    uint32_t rd_off = 0;  // byte offset of the stage being multiplied
    // fetch_c: read the fragments of the following step; issue_c: this step carries DMA;
    // wait_c: vmcnt bound to wait for before crossing into the next slab (-1: no crossing wait)
    auto step = [&](auto kk_c, auto fetch_c, auto issue_c, auto wait_c, const uint32_t next_off, const KUnit ku) {
        constexpr int kk = decltype(kk_c)::value;
        constexpr bool fetch = decltype(fetch_c)::value, issue = decltype(issue_c)::value;
        constexpr int waitn = decltype(wait_c)::value;
        constexpr int cur = kk & 1, nxt = cur ^ 1;
        constexpr bool cross = kk == KSTEPS - 1;  // the following step belongs to the next slab
        constexpr int w = (kk + 1) % KSTEPS;      // position of this step in the DMA window, which opens at the crossing
        typedef std::integral_constant<int, cur> cur_c;
        typedef std::integral_constant<int, nxt> nxt_c;
        static_for<NMF>([&](auto q_c) {
            constexpr int q = decltype(q_c)::value, i = q / FN, jj = q % FN;
            acc[i][jj] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[cur][jj], af[cur][i], acc[i][jj], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (fetch) {
                if constexpr (cross && q == 0) {
                    wait_vmcnt<waitn>();
                    __syncthreads();
                }
                static_for<RPS>([&](auto t_c) {
                    constexpr int r = q * RPS + decltype(t_c)::value;
                    if constexpr (r < NREADS) {
                        if constexpr (cross)
                            read_frag(std::integral_constant<int, r>{}, nxt_c{}, stages + next_off, 0);
                        else
                            read_frag(std::integral_constant<int, r>{}, nxt_c{}, stages + rd_off, (kk + 1) * 2);
                    }
                });
            }
            if constexpr (issue && w < WINDOW) {
                static_for<DPS>([&](auto t_c) {
                    constexpr int idx = (w * NMF + q) * DPS + decltype(t_c)::value;
                    // the buffer being refilled is the one whose last fragments were read a step ago
                    if constexpr (idx < LPS) issue_piece(std::integral_constant<int, idx>{}, cross ? rd_off : next_off, ku);
                });
            }
            if constexpr (q == NMF - 1) {
                if constexpr (fetch) flip(nxt_c{}, c0{});
            } else if constexpr ((q + 1) % FN == 0) {
                flip(cur_c{}, std::integral_constant<int, (q + 1) / FN>{});
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    typedef std::true_type yes;
    typedef std::false_type no;

    if (k_slabs >= STAGES)
        wait_vmcnt<(STAGES - 1) * LPS>();
    else
        wait_vmcnt<0>();
    __syncthreads();
    static_for<NREADS>([&](auto r_c) { read_frag(r_c, c0{}, stages, 0); });
    flip(c0{}, c0{});
    // steps 0 .. KSTEPS-2 of slab 0
    static_for<KSTEPS - 1>([&](auto kk_c) { step(kk_c, yes{}, no{}, no_wait{}, 0u, KUnit()); });
    // iteration `it`: last step of slab it, then steps 0 .. KSTEPS-2 of slab it+1
    int it = 0;
    for (; it < k_slabs - STAGES; ++it) {
        KUnit ku = tail_unit(it + STAGES);
        if constexpr (!DENSE) ku = ktab_s[(it + STAGES) * CPR + my_chunk];
        const uint32_t freed = rd_off;
        const uint32_t next_off = rd_off + STAGE_BYTES == STAGES * STAGE_BYTES ? 0u : rd_off + STAGE_BYTES;
        step(std::integral_constant<int, KSTEPS - 1>{}, yes{}, yes{}, std::integral_constant<int, (STAGES - 2) * LPS>{}, next_off, ku);
        rd_off = next_off;
        // in the steps after the crossing, `freed` is what the crossing step called rd_off
        static_for<KSTEPS - 1>([&](auto kk_c) { step(kk_c, yes{}, yes{}, no_wait{}, freed, ku); });
        advance_slab();
    }
    for (; it < k_slabs - 1; ++it) {  // the last stages are in flight: nothing more to issue
        const uint32_t next_off = rd_off + STAGE_BYTES == STAGES * STAGE_BYTES ? 0u : rd_off + STAGE_BYTES;
        step(std::integral_constant<int, KSTEPS - 1>{}, yes{}, no{}, c0{}, next_off, KUnit());
        rd_off = next_off;
        static_for<KSTEPS - 1>([&](auto kk_c) { step(kk_c, yes{}, no{}, no_wait{}, 0u, KUnit()); });
    }
    step(std::integral_constant<int, KSTEPS - 1>{}, no{}, no{}, no_wait{}, 0u, KUnit());

    // ---- epilogue.  acc[i][j][r] belongs to pixel row i*32 + (lane & 31) and, with the row
    // permutation of the packed weights, channel j*32 + 16*(lane >> 5) + r of this wave's sub-tile.
    if constexpr (ROWSUM) {
        if (wn == 0) {
#pragma unroll
            for (int i = 0; i < FM; ++i) rowsum_s[wk * 2 + fhalf][wm * WTM + i * 32 + frow] = rowsum[i];
        }
    }
    if (tid < BN) bias_s[tid] = bias_reg;
    __syncthreads();  // row sums and bias visible; every wave is done with the operand stages
    const RequantDev rq = p.rq;

    if constexpr (WGK == 1) {
        size_t row_off[FM];
        int ncorr[FM];
        bool row_ok[FM];
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            const int ml = wm * WTM + i * 32 + frow, m = m0 + ml;
            row_ok[i] = m < p.m;
            row_off[i] = row_ok[i] ? out_pixel_offset(p, m, plane) : 0;
            ncorr[i] = ROWSUM ? -p.zw * (rowsum_s[0][ml] + rowsum_s[1][ml]) : 0;
        }
        // whole tiles with 16-byte aligned rows (the usual case) store without any per-store test
        const bool aligned16 = (p.ldc & 15) == 0 && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
        auto emit = [&](auto checked_c, auto fast_c, auto pc_c) {
            constexpr bool checked = decltype(checked_c)::value;
            constexpr int fast = decltype(fast_c)::value;
            constexpr bool pc = decltype(pc_c)::value;  // one multiplier and shift per channel
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                const int nl = wn * WTN + j * 32 + fhalf * 16, n = n0 + nl;  // this lane's 16 consecutive channels
                if constexpr (checked) {
                    if (n >= p.n) continue;  // past the last channel: nothing to requantize
                }
                int4 bb[4];
#pragma unroll
                for (int g = 0; g < 4; ++g) bb[g] = *reinterpret_cast<const int4 *>(bias_s + nl + g * 4);
                int4 cm[pc ? 4 : 1], cs[pc ? 4 : 1];
                if constexpr (pc) {  // the arrays are padded past the last channel block
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        cm[g] = *reinterpret_cast<const int4 *>(rq.pc_multiplier + n + g * 4);
                        cs[g] = *reinterpret_cast<const int4 *>(rq.pc_shift + n + g * 4);
                    }
                }
#pragma unroll
                for (int i = 0; i < FM; ++i) {
                    uint32_t packed[4];
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        uint32_t o0, o1, o2, o3;
                        if constexpr (pc && fast != 0) {  // every channel's pair inside the single-shift form's range
                            o0 = requant_u8_channel_fast<fast>(acc[i][j][g * 4 + 0] + bb[g].x + ncorr[i], cm[g].x, cs[g].x, rq);
                            o1 = requant_u8_channel_fast<fast>(acc[i][j][g * 4 + 1] + bb[g].y + ncorr[i], cm[g].y, cs[g].y, rq);
                            o2 = requant_u8_channel_fast<fast>(acc[i][j][g * 4 + 2] + bb[g].z + ncorr[i], cm[g].z, cs[g].z, rq);
                            o3 = requant_u8_channel_fast<fast>(acc[i][j][g * 4 + 3] + bb[g].w + ncorr[i], cm[g].w, cs[g].w, rq);
                        } else if constexpr (pc) {
                            o0 = requant_u8_channel(acc[i][j][g * 4 + 0] + bb[g].x + ncorr[i], cm[g].x, cs[g].x, rq);
                            o1 = requant_u8_channel(acc[i][j][g * 4 + 1] + bb[g].y + ncorr[i], cm[g].y, cs[g].y, rq);
                            o2 = requant_u8_channel(acc[i][j][g * 4 + 2] + bb[g].z + ncorr[i], cm[g].z, cs[g].z, rq);
                            o3 = requant_u8_channel(acc[i][j][g * 4 + 3] + bb[g].w + ncorr[i], cm[g].w, cs[g].w, rq);
                        } else if constexpr (fast != 0) {
                            packed[g] = requant4_fast<fast>(acc[i][j][g * 4 + 0] + bb[g].x, acc[i][j][g * 4 + 1] + bb[g].y,
                                                            acc[i][j][g * 4 + 2] + bb[g].z, acc[i][j][g * 4 + 3] + bb[g].w, ncorr[i], rq) ^
                                        p.out_xor;
                            continue;
                        } else {
                            o0 = requant_u8_as<fast>(acc[i][j][g * 4 + 0] + bb[g].x + ncorr[i], rq);
                            o1 = requant_u8_as<fast>(acc[i][j][g * 4 + 1] + bb[g].y + ncorr[i], rq);
                            o2 = requant_u8_as<fast>(acc[i][j][g * 4 + 2] + bb[g].z + ncorr[i], rq);
                            o3 = requant_u8_as<fast>(acc[i][j][g * 4 + 3] + bb[g].w + ncorr[i], rq);
                        }
                        packed[g] = pack_bytes(o0, o1, o2, o3) ^ p.out_xor;
                    }
                    uint8_t *dst = p.out + row_off[i] + n;
                    if constexpr (!checked) {
                        *reinterpret_cast<uint4 *>(dst) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
                        __builtin_amdgcn_sched_barrier(0);  // one fragment at a time: keeps the accumulators where they are
                    } else {
                        if (!row_ok[i]) continue;
                        if (aligned16 && n + 16 <= p.n) {
                            *reinterpret_cast<uint4 *>(dst) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
                        } else {
                            if constexpr (BM == 256 && BN == 256) {  // (no registers to spare for the dword form's copies)
                                const int cnt = p.n - n < 16 ? p.n - n : 16;
                                for (int t = 0; t < cnt; ++t) dst[t] = (uint8_t)(packed[t >> 2] >> (8 * (t & 3)));
                            } else {
                                store_bytes_any_alignment(dst, packed, p.n - n < 16 ? p.n - n : 16);
                            }
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        };
        // edge tiles and unusual requantization parameters take the general code
        if (rq.pc_multiplier) {
            // (the 256 x 256 tile has no registers to spare for the per-channel terms: two-step order there)
            constexpr bool pc_single_shift = !(BM == 256 && BN == 256);
            if (pc_single_shift && rq.fast == 2)
                emit(std::true_type{}, std::integral_constant<int, pc_single_shift ? 2 : 0>{}, std::true_type{});
            else if (pc_single_shift && rq.fast == 1)
                emit(std::true_type{}, std::integral_constant<int, pc_single_shift ? 1 : 0>{}, std::true_type{});
            else
                emit(std::true_type{}, std::integral_constant<int, 0>{}, std::true_type{});
        } else if (rq.fast && aligned16 && m0 + BM <= p.m && n0 + BN <= p.n) {
            if (rq.fast == 2)
                emit(std::false_type{}, std::integral_constant<int, 2>{}, std::false_type{});
            else
                emit(std::false_type{}, std::integral_constant<int, 1>{}, std::false_type{});
        } else if (rq.fast == 2) {  // edge tiles (and layers narrower than the tile) keep the short requantization forms
            emit(std::true_type{}, std::integral_constant<int, 2>{}, std::false_type{});
        } else if (rq.fast == 1) {
            emit(std::true_type{}, std::integral_constant<int, 1>{}, std::false_type{});
        } else {
            emit(std::true_type{}, std::integral_constant<int, 0>{}, std::false_type{});
        }
    } else {
        // the WGK partial tiles meet in LDS: [wk][pixel row][channel], rows padded so that
        // eight consecutive rows of 16-byte accesses fall in distinct banks
        int32_t *part = reinterpret_cast<int32_t *>(stages) + wk * BM * PART_ROW;
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    int4 v;
                    v.x = acc[i][j][g * 4 + 0];
                    v.y = acc[i][j][g * 4 + 1];
                    v.z = acc[i][j][g * 4 + 2];
                    v.w = acc[i][j][g * 4 + 3];
                    *reinterpret_cast<int4 *>(part + (i * 32 + frow) * PART_ROW + j * 32 + fhalf * 16 + g * 4) = v;
                }
        __syncthreads();
        // thread -> pixel row tid & 63, sixteen channels starting at (tid >> 6) * 16
        const int ml = tid & 63, nl = (tid >> 6) * 16;
        const int m = m0 + ml, n = n0 + nl;
        if (m >= p.m || n >= p.n) return;
        int corr = 0;
        if constexpr (ROWSUM) {
#pragma unroll
            for (int w = 0; w < WGK * 2; ++w) corr += rowsum_s[w][ml];
            corr *= p.zw;
        }
        const int32_t *pr = reinterpret_cast<const int32_t *>(stages) + ml * PART_ROW + nl;
        if (p.partial) {  // a slice of a reduction shared between workgroups: the sums leave as they are
            int32_t *dst = p.partial + ((size_t)m * (size_t)p.partial_ld + (size_t)n);
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                int4 s4 = *reinterpret_cast<const int4 *>(pr + g * 4);
#pragma unroll
                for (int w = 1; w < WGK; ++w) {
                    const int4 t = *reinterpret_cast<const int4 *>(pr + g * 4 + w * BM * PART_ROW);
                    s4.x += t.x;
                    s4.y += t.y;
                    s4.z += t.z;
                    s4.w += t.w;
                }
                *reinterpret_cast<int4 *>(dst + g * 4) = make_int4(s4.x - corr, s4.y - corr, s4.z - corr, s4.w - corr);
            }
            return;
        }
        uint32_t packed[4];
        auto reduce = [&](auto fast_c) {
            constexpr int fast = decltype(fast_c)::value;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            int4 s4 = *reinterpret_cast<const int4 *>(pr + g * 4);
#pragma unroll
            for (int w = 1; w < WGK; ++w) {
                const int4 t = *reinterpret_cast<const int4 *>(pr + g * 4 + w * BM * PART_ROW);
                s4.x += t.x;
                s4.y += t.y;
                s4.z += t.z;
                s4.w += t.w;
            }
            const int4 bb = *reinterpret_cast<const int4 *>(bias_s + nl + g * 4);
            uint32_t o0, o1, o2, o3;
            if (rq.pc_multiplier) {
                const int32_t *pm = rq.pc_multiplier + n + g * 4;
                const int4 cm = make_int4(pm[0], pm[1], pm[2], pm[3]);
                const int32_t *ps = rq.pc_shift + n + g * 4;
                const int4 cs = make_int4(ps[0], ps[1], ps[2], ps[3]);
                if constexpr (fast != 0) {
                    o0 = requant_u8_channel_fast<fast>(s4.x + bb.x - corr, cm.x, cs.x, rq);
                    o1 = requant_u8_channel_fast<fast>(s4.y + bb.y - corr, cm.y, cs.y, rq);
                    o2 = requant_u8_channel_fast<fast>(s4.z + bb.z - corr, cm.z, cs.z, rq);
                    o3 = requant_u8_channel_fast<fast>(s4.w + bb.w - corr, cm.w, cs.w, rq);
                } else {
                    o0 = requant_u8_channel(s4.x + bb.x - corr, cm.x, cs.x, rq);
                    o1 = requant_u8_channel(s4.y + bb.y - corr, cm.y, cs.y, rq);
                    o2 = requant_u8_channel(s4.z + bb.z - corr, cm.z, cs.z, rq);
                    o3 = requant_u8_channel(s4.w + bb.w - corr, cm.w, cs.w, rq);
                }
            } else if constexpr (fast != 0) {
                packed[g] = requant4_fast<fast>(s4.x + bb.x, s4.y + bb.y, s4.z + bb.z, s4.w + bb.w, -corr, rq) ^ p.out_xor;
                continue;
            } else {
                o0 = requant_u8_as<fast>(s4.x + bb.x - corr, rq), o1 = requant_u8_as<fast>(s4.y + bb.y - corr, rq);
                o2 = requant_u8_as<fast>(s4.z + bb.z - corr, rq), o3 = requant_u8_as<fast>(s4.w + bb.w - corr, rq);
            }
            packed[g] = pack_bytes(o0, o1, o2, o3) ^ p.out_xor;
        }
        };
        if (rq.fast == 2)
            reduce(std::integral_constant<int, 2>{});
        else if (rq.fast == 1)
            reduce(std::integral_constant<int, 1>{});
        else
            reduce(std::integral_constant<int, 0>{});
        const size_t out_off = out_pixel_offset(p, m, plane) + n;
        uint8_t *dst = p.out + out_off;
        const bool aligned16 = (p.ldc & 15) == 0 && ((reinterpret_cast<uintptr_t>(p.out) & 15) == 0);
        if (p.residual) {  // out = add(residual, result); only this split-reduction epilogue offers it
            const uint8_t *res = p.residual + out_off;
            if (res_vec) {
                const uint4 rv = res_reg;
                // add_word with the two tables (the same arithmetic: the tables hold what add_one computes first)
                auto add_word_lut = [&](uint32_t a, uint32_t b) {
                    uint32_t o = 0;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int32_t sum = add_lut_s[0][(a >> (8 * i)) & 255u] + add_lut_s[1][(b >> (8 * i)) & 255u];
                        int32_t v = mul_round_shift(sum, p.radd.mult_out, p.radd.rs_out) + p.radd.zp_out;
                        v = v < p.radd.act_min ? p.radd.act_min : v;
                        v = v > p.radd.act_max ? p.radd.act_max : v;
                        o |= (uint32_t)v << (8 * i);
                    }
                    return o;
                };
                packed[0] = add_word_lut(rv.x, packed[0]);
                packed[1] = add_word_lut(rv.y, packed[1]);
                packed[2] = add_word_lut(rv.z, packed[2]);
                packed[3] = add_word_lut(rv.w, packed[3]);
            } else {
                const int cnt = p.n - n < 16 ? p.n - n : 16;
                for (int t = 0; t < cnt; ++t) {
                    const uint32_t v = add_one(res[t], (packed[t >> 2] >> (8 * (t & 3))) & 255u, p.radd);
                    packed[t >> 2] = (packed[t >> 2] & ~(255u << (8 * (t & 3)))) | (v << (8 * (t & 3)));
                }
            }
        }
        if (aligned16 && n + 16 <= p.n) {
            *reinterpret_cast<uint4 *>(dst) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
        } else {
            store_bytes_any_alignment(dst, packed, p.n - n < 16 ? p.n - n : 16);
        }
    }
}

template <int BM, int BN, int WGM, int WGN, int WGK, int SLAB, int STAGES>
int launch_cfg(const GemmProblem *ps, int count, hipStream_t stream) {
    const GemmProblem &p = ps[0];
    GemmBatch batch;
    for (int i = 0; i < count; ++i) batch.p[i] = ps[i];
    static_assert(STAGES * (BM + BN) * SLAB + WGK * 2 * BM * 4 + BN * 4 <= 160 * 1024 - 12288, "LDS budget with the largest k-table");
    int m_max = p.m;  // (table-driven problems of one launch may differ in their row counts: every kernel tests rows against its own problem's)
    for (int i = 1; i < count; ++i) m_max = ps[i].m > m_max ? ps[i].m : m_max;
    const int tiles_m = (m_max + BM - 1) / BM, tiles_n = (p.n + BN - 1) / BN;
    // group size: 32 tiles, or fewer (a power of two) when that is needed to give each of the 8 XCDs a group
    int gs = 32;
    while (gs > 1 && (long)tiles_m * tiles_n * count < 8l * gs) gs >>= 1;
    // group shape gm x gn: least operand rows per group among the shapes that fit the tile grid
    int gm = 1;
    long best = -1;
    for (int cand = 1; cand <= gs; cand *= 2) {
        const int gn = gs / cand;
        const long cost = (long)(cand < tiles_m ? cand : tiles_m) * BM + (long)(gn < tiles_n ? gn : tiles_n) * BN;
        const long waste = (long)((tiles_m + cand - 1) / cand) * ((tiles_n + gn - 1) / gn);  // groups launched
        const long score = cost * waste;
        if (best < 0 || score < best) {
            best = score;
            gm = cand;
        }
    }
    int gn = gs / gm;
    const int groups = ((tiles_m + gm - 1) / gm) * ((tiles_n + gn - 1) / gn) * count;
    int grid = ((groups + 7) / 8) * 8 * gs;
    // rectangles that overhang the tile grid leave workgroup slots empty; where that costs a launch of up to a few
    // rounds more than an eighth of its slots, split the tiles evenly over the XCDs instead
    const long tiles_all = (long)tiles_m * tiles_n * count;
    if (tiles_all <= 1024 && (long)grid * 8 > tiles_all * 9) {
        gm = 0;
        gn = (int)((tiles_all + 7) / 8);  // tiles per XCD
        grid = gn * 8;
    }
    const size_t ktab_bytes = (size_t)(p.k_pad / 16) * sizeof(KUnit);
    // the per-row activation sums are only carried when the weight zero point is not 128
    // a plain matrix whose reduction ends inside its last slab has a kernel variant of its own where the 64 x 64 tile
    // with the split reduction serves it (1x1 layers with 320 .. 960 input channels); elsewhere it is gathered by table
    constexpr bool ragged_variant = BM == 64 && BN == 64;
    const bool whole = p.k == p.k_pad;
    if (p.dense && whole) {
        if (p.zw != 0)
            hipLaunchKernelGGL((igemm_dma_kernel<BM, BN, WGM, WGN, WGK, SLAB, STAGES, 1, true>), dim3(grid), dim3(256), 0,
                               stream, batch, count, tiles_m, tiles_n, gm, gn);
        else
            hipLaunchKernelGGL((igemm_dma_kernel<BM, BN, WGM, WGN, WGK, SLAB, STAGES, 1, false>), dim3(grid), dim3(256), 0,
                               stream, batch, count, tiles_m, tiles_n, gm, gn);
    } else if (p.dense && ragged_variant) {
        if constexpr (ragged_variant) {
            if (p.zw != 0)
                hipLaunchKernelGGL((igemm_dma_kernel<BM, BN, WGM, WGN, WGK, SLAB, STAGES, 2, true>), dim3(grid), dim3(256), 0,
                                   stream, batch, count, tiles_m, tiles_n, gm, gn);
            else
                hipLaunchKernelGGL((igemm_dma_kernel<BM, BN, WGM, WGN, WGK, SLAB, STAGES, 2, false>), dim3(grid), dim3(256), 0,
                                   stream, batch, count, tiles_m, tiles_n, gm, gn);
        }
    } else {
        if (p.zw != 0)
            hipLaunchKernelGGL((igemm_dma_kernel<BM, BN, WGM, WGN, WGK, SLAB, STAGES, 0, true>), dim3(grid), dim3(256),
                               ktab_bytes, stream, batch, count, tiles_m, tiles_n, gm, gn);
        else
            hipLaunchKernelGGL((igemm_dma_kernel<BM, BN, WGM, WGN, WGK, SLAB, STAGES, 0, false>), dim3(grid), dim3(256),
                               ktab_bytes, stream, batch, count, tiles_m, tiles_n, gm, gn);
    }
    EH_HIP(hipGetLastError());
    return EH_OK;
}

// Adds up the slices of a reduction that several workgroups shared and finishes the outputs: bias, requantization in
// the reference's own order (the single-shift forms the epilogues use are its equivalents), the residual add, the store.
// One thread per output pixel and sixteen channels.
__global__ __launch_bounds__(256) void splitk_finish_kernel(const GemmProblem p, const int32_t *__restrict__ partial, const int partial_ld,
                                                            const int slices, const int chunks, const FastDiv div_chunks) {
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    const int m = (int)fastdiv(idx, div_chunks), n = ((int)idx - m * chunks) * 16;
    if (m >= p.m) return;
    const size_t slice_stride = (size_t)p.m * (size_t)partial_ld;
    const int32_t *src = partial + ((size_t)m * (size_t)partial_ld + (size_t)n);
    const RequantDev rq = p.rq;
    uint32_t packed[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        int4 v = *reinterpret_cast<const int4 *>(p.bias + n + g * 4);
        for (int s = 0; s < slices; ++s) {
            const int4 t = *reinterpret_cast<const int4 *>(src + s * slice_stride + g * 4);
            v.x += t.x;
            v.y += t.y;
            v.z += t.z;
            v.w += t.w;
        }
        uint32_t o0, o1, o2, o3;
        if (rq.pc_multiplier) {
            const int4 cm = *reinterpret_cast<const int4 *>(rq.pc_multiplier + n + g * 4), cs = *reinterpret_cast<const int4 *>(rq.pc_shift + n + g * 4);
            o0 = requant_u8_channel(v.x, cm.x, cs.x, rq), o1 = requant_u8_channel(v.y, cm.y, cs.y, rq);
            o2 = requant_u8_channel(v.z, cm.z, cs.z, rq), o3 = requant_u8_channel(v.w, cm.w, cs.w, rq);
        } else {
            o0 = requant_u8(v.x, rq), o1 = requant_u8(v.y, rq), o2 = requant_u8(v.z, rq), o3 = requant_u8(v.w, rq);
        }
        packed[g] = pack_bytes(o0, o1, o2, o3) ^ p.out_xor;
    }
    const int cnt = p.n - n < 16 ? p.n - n : 16;
    const size_t out_off = out_pixel_offset(p, m, p.ho * p.wo) + (size_t)n;
    if (p.residual) {
        const uint8_t *res = p.residual + out_off;
        for (int t = 0; t < cnt; ++t) {
            const uint32_t v = add_one(res[t], (packed[t >> 2] >> (8 * (t & 3))) & 255u, p.radd);
            packed[t >> 2] = (packed[t >> 2] & ~(255u << (8 * (t & 3)))) | (v << (8 * (t & 3)));
        }
    }
    uint8_t *dst = p.out + out_off;
    if (cnt == 16 && (p.ldc & 15) == 0 && (reinterpret_cast<uintptr_t>(p.out) & 15) == 0)
        *reinterpret_cast<uint4 *>(dst) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
    else
        store_bytes_any_alignment(dst, packed, cnt);
}

}  // namespace

int launch_splitk_finish(const GemmProblem &p, const int32_t *partial, int32_t partial_ld, int32_t slices, hipStream_t stream) {
    EH_REQUIRE(partial != nullptr && slices >= 1 && partial_ld >= (p.n + 15) / 16 * 16 && (partial_ld & 3) == 0, "splitk_finish: bad partial image");
    const int chunks = (p.n + 15) / 16;
    const long total = (long)p.m * chunks;
    if (total <= 0) return EH_OK;
    EH_REQUIRE(total < (1l << 31), "splitk_finish: too many outputs");
    hipLaunchKernelGGL(splitk_finish_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, p, partial, partial_ld, slices, chunks,
                       make_fastdiv((uint32_t)chunks));
    EH_HIP(hipGetLastError());
    return EH_OK;
}

// Which kernel shape serves an (m, n, k) problem whose activations come in
// 16-byte channel units.  The packed weight layout depends on the slab, so the
// choice is made once, when the weights are packed.
// `siblings` equally shaped problems share one launch (convolution groups, deconvolution phases).
GemmConfig igemm_dma_select(int32_t m, int32_t n, int32_t k, int32_t siblings) {
    GemmConfig c;
    const long t256 = (long)((m + 255) / 256) * ((n + 127) / 128) * siblings;
    const long t128 = (long)((m + 127) / 128) * ((n + 127) / 128) * siblings;
    const long t128x64 = (long)((m + 127) / 128) * ((n + 63) / 64) * siblings;
    const long t256x256 = (long)((m + 255) / 256) * ((n + 255) / 256) * siblings;
    if (n > 128 && t256x256 >= 240) {
        c.id = GEMM_DMA_256x256;
        c.slab = 128;
    } else if (n > 64 && t256 >= 240) {
        c.id = GEMM_DMA_256x128;
        c.slab = 128;
    } else if (n > 64 && t128 > 128) {
        // (more than 128 of these are more than 512 split-reduction tiles, i.e. three of those per CU on some CUs: from there
        // on one round of 128 x 128 tiles is as fast or faster at every reduction length measured, 1.5x at 18 KiB; up to
        // 128 the split-reduction tiles win, 17.9 against 26.0 us at 100 tiles and a 4.5 KiB reduction)
        c.id = GEMM_DMA_128x128;
        c.slab = 128;
    } else if (n <= 64 && t128x64 >= 200) {
        c.id = GEMM_DMA_128x64;
        c.slab = 128;
    } else {
        c.id = GEMM_DMA_64x64_SPLITK;
        c.slab = 256;
    }
    (void)k;
    return c;
}

int launch_igemm_dma(const GemmProblem *ps, int count, hipStream_t stream) {
    const GemmProblem &p = ps[0];
    EH_REQUIRE(count >= 1 && count <= GemmBatch::MAX, "igemm_dma: batch of %d", count);
    for (int i = 0; i < count; ++i) {
        EH_REQUIRE(ps[i].vec == 16 && ps[i].k_pad % ps[i].cfg.slab == 0, "igemm_dma: unsupported problem");
        EH_REQUIRE(ps[i].cfg.id == p.cfg.id && (ps[i].m == p.m || (!p.dense && !p.partial)) && ps[i].n == p.n && ps[i].k_pad == p.k_pad &&
                       ps[i].dense == p.dense && ps[i].zw == p.zw,
                   "igemm_dma: a batch must hold equally shaped problems");
    }
    switch (p.cfg.id) {
        case GEMM_DMA_256x256: return launch_cfg<256, 256, 2, 2, 1, 128, 2>(ps, count, stream);
        case GEMM_DMA_256x128: return launch_cfg<256, 128, 2, 2, 1, 128, 3>(ps, count, stream);
        case GEMM_DMA_128x128: return launch_cfg<128, 128, 2, 2, 1, 128, 2>(ps, count, stream);
        case GEMM_DMA_128x64: return launch_cfg<128, 64, 4, 1, 1, 128, 2>(ps, count, stream);
        case GEMM_DMA_64x64_SPLITK: {
            // Two stages take half the LDS, so two workgroups share a CU: for reductions of one or two slabs (deeper
            // staging has nothing to prefetch) and for launches with more tiles than CUs (the second workgroup's
            // prologue and epilogue hide behind the first one's loop instead of forming a second round).
            int m_max = p.m;
            for (int i = 1; i < count; ++i) m_max = ps[i].m > m_max ? ps[i].m : m_max;
            const long tiles = (long)((m_max + 63) / 64) * ((p.n + 63) / 64) * count;
            if (p.k_pad / 256 <= 2 || tiles > 256) return launch_cfg<64, 64, 1, 1, 4, 256, 2>(ps, count, stream);
            return launch_cfg<64, 64, 1, 1, 4, 256, 4>(ps, count, stream);
        }
        default: break;
    }
    set_error("igemm_dma: unknown configuration %d", p.cfg.id);
    return EH_INVALID_PARAMS;
}

}  // namespace eh
