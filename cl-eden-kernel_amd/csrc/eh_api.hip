// C ABI of libedenhip.so: host arithmetic, device buffers, and the operator
// plans (packed weights + folded bias + k-tables) behind eden_hip.h.
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <new>
#include <vector>

#include "eh_internal.h"

namespace eh {

// ------------------------------------------------------------------ errors
static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int hip_fail(hipError_t e, const char *what) {
    set_error("%s: %s", what, hipGetErrorString(e));
    return EH_DEVICE_FAILURE;
}

// ------------------------------------------------------------------ static scratch
// Device memory for the entry point that may not allocate (eh_conv2d_u8_run_static): one array per GPU, part of the
// code object, held from the moment the library is loaded on a device until the process ends.  In host code the
// array's name is only a handle for hipGetSymbolAddress; `static_scratch` asks once per device, with that device
// current, and every later use (kernel arguments, copies) goes through the address it keeps.
static __device__ __align__(256) uint8_t scratch[EH_STATIC_SCRATCH_BYTES];
static constexpr int kMaxDevices = 64;
// longest reduction (channels x kernel taps, or the columns of a fully connected layer) a plan is built for:
// the per-plan tables grow with it, and no layer of the networks this serves comes near it
static constexpr int EH_MAX_REDUCTION = 1 << 24;
static uint8_t *g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each device, null until asked

static int static_scratch(uint8_t **ptr) {
    int dev = -1;
    EH_HIP(hipGetDevice(&dev));
    EH_REQUIRE(dev >= 0 && dev < kMaxDevices, "device ordinal %d is outside the static scratch table", dev);
    uint8_t *p = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
    if (p == nullptr) {
        void *addr = nullptr;
        EH_HIP(hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch)));
        EH_REQUIRE(addr != nullptr, "hipGetSymbolAddress returned a null address for the static scratch");
        p = static_cast<uint8_t *>(addr);
        __atomic_store_n(&g_scratch_ptr[dev], p, __ATOMIC_RELEASE);  // concurrent first calls store the same address
    }
    *ptr = p;
    return EH_OK;
}

// int8 tensors are computed as their uint8 equivalents: every stored value, zero point and clamp bound + 128
// (SIGNED_TO_UNSIGNED in gpu/operators/cl_kernels/DepthwiseconvolutionKernels.cpp:2410-2411, and the zero points
// + 128 of cl_optimized_impls/CLDepthwiseConvolutionQuantized.cpp:207-211)
static eh_requant io_as_uint8(const eh_requant &q) {
    eh_requant u = q;
    u.zp_in += 128;
    u.zp_out += 128;
    u.act_min += 128;
    u.act_max += 128;
    return u;
}

int check_requant(const eh_requant *q, bool signed_weights, bool signed_io) {
    EH_REQUIRE(q != nullptr, "requant parameters are null");
    if (signed_weights) {
        EH_REQUIRE(q->zp_w >= -128 && q->zp_w <= 127, "int8 weight zero point %d outside [-128, 127]", q->zp_w);
        eh_requant u = *q;
        u.zp_w += 128;
        return check_requant(&u, false, signed_io);
    }
    if (signed_io) {
        EH_REQUIRE(q->zp_in >= -128 && q->zp_in <= 127, "int8 input zero point %d outside [-128, 127]", q->zp_in);
        EH_REQUIRE(q->act_min >= -128 && q->act_max <= 127 && q->act_min <= q->act_max, "int8 activation range [%d, %d] invalid",
                   q->act_min, q->act_max);
        const eh_requant u = io_as_uint8(*q);
        return check_requant(&u, false, false);
    }
    EH_REQUIRE(q->multiplier >= 0, "requant multiplier %d is negative", q->multiplier);
    EH_REQUIRE(q->shift >= -31 && q->shift <= 30, "requant shift %d outside [-31, 30]", q->shift);
    EH_REQUIRE(q->zp_in >= 0 && q->zp_in <= 255 && q->zp_w >= 0 && q->zp_w <= 255,
               "uint8 zero points (%d, %d) outside [0, 255]", q->zp_in, q->zp_w);
    EH_REQUIRE(q->act_min >= 0 && q->act_max <= 255 && q->act_min <= q->act_max, "activation range [%d, %d] invalid",
               q->act_min, q->act_max);
    return EH_OK;
}

namespace {

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }
inline int round_up(int v, int a) { return (v + a - 1) / a * a; }

// Set while a descriptor is only being asked which kernels would serve it: geometry and kernel choice are
// computed as for a plan, nothing is allocated or copied.
static thread_local bool g_dry_run = false;

template <typename T>
int dev_alloc(T **p, size_t count) {
    *p = nullptr;
    if (g_dry_run) return EH_OK;
    if (count == 0) count = 1;
    EH_HIP(hipMalloc(reinterpret_cast<void **>(p), count * sizeof(T)));
    return EH_OK;
}

template <typename T>
void dev_free(T *&p) {
    if (p) (void)hipFree(p);
    p = nullptr;
}

// One GEMM the operator decomposes into: a convolution group or a
// deconvolution output phase.
struct GemmPart {
    int8_t *b = nullptr;
    int32_t *colsum = nullptr;
    int32_t *folded = nullptr;
    KUnit *ktab = nullptr;
    int32_t *tap_off = nullptr;
    int32_t n = 0, n_pad = 0, k = 0, k_pad = 0, vec = 1, taps = 0, cin = 0;
    int32_t cin_real = 0;     // channels per tap in the source weights when `cin` includes padding channels; 0 = cin
    // Several kernel columns of a transposed convolution as one problem (their outputs are neighbouring pixels): column
    // o of the problem is output channel o % n_period of kernel column o / n_period, `period_step` weight elements on.
    int32_t n_period = 0;
    int64_t period_step = 0;
    int32_t *pc_multiplier_rep = nullptr, *pc_shift_rep = nullptr;  // the operator's per-channel pairs, repeated per kernel column
    // Few output tiles under a long reduction: `slices` workgroups share each tile's reduction (equal runs of slabs) and
    // leave int32 sums in `partial` [slices][m][n_pad], which a second small launch adds up and requantizes.
    int32_t slices = 0;
    int32_t *partial = nullptr;
    // Several convolution groups as one block-diagonal problem (channels per group below 16): `block_cin` input and
    // `block_n` output channels per group; the entries off the blocks hold the weight zero point, so they are packed
    // again from the operator's copy of the weights whenever that changes.
    int32_t block_cin = 0, block_n = 0;
    GemmConfig cfg;
    int64_t so = 0, sc = 0;   // source weight strides (out channel, in channel)
    int64_t w_base = 0;       // element offset of this part in the source weights
    int32_t bias_base = 0;    // first output channel
    GemmProblem proto{};      // geometry; pointers and quantization filled per run

    void release() {
        dev_free(b);
        dev_free(colsum);
        dev_free(folded);
        dev_free(ktab);
        dev_free(tap_off);
        dev_free(pc_multiplier_rep);
        dev_free(pc_shift_rep);
        dev_free(partial);
    }
};

int pick_vec(int cig, int pixel_stride) {
    if ((cig & 15) == 0 && (pixel_stride & 15) == 0) return 16;
    if ((cig & 3) == 0 && (pixel_stride & 3) == 0) return 4;
    return 1;
}

// whether the load units describe the nine taps of a 3x3 window at dilation 1, row by row, `per_tap` units each
static bool units_are_3x3(const std::vector<KUnit> &units, int per_tap) {
    if (per_tap <= 0 || units.size() != (size_t)9 * per_tap) return false;
    for (int t = 0; t < 9; ++t)
        if (units[(size_t)t * per_tap].dy != t / 3 || units[(size_t)t * per_tap].dx != t % 3) return false;
    return true;
}

// Whether the load units describe kh x kw taps at dilation 1, row by row, `per_tap` units each; kw = the taps of row 0.
static bool units_are_rows(const std::vector<KUnit> &units, int per_tap, int taps, int &kh, int &kw) {
    if (per_tap <= 0 || taps <= 0 || units.size() != (size_t)taps * per_tap) return false;
    kw = 0;
    while (kw < taps && units[(size_t)kw * per_tap].dy == 0) ++kw;
    if (kw == 0 || taps % kw != 0) return false;
    kh = taps / kw;
    for (int t = 0; t < taps; ++t)
        if (units[(size_t)t * per_tap].dy != t / kw || units[(size_t)t * per_tap].dx != t % kw) return false;
    return true;
}

// Allocates a part's device arrays and uploads its tables.  `units` holds one
// KUnit per `vec` bytes of the real reduction length; padding units are added here.
// k_floor > 0: the part is one of several whose reductions differ in length and that should share a launch: its
// reduction is padded to k_floor (the padding units read a constant that multiplies to zero) and only the tiled
// kernels are considered, so that every sibling gets the same configuration.
int finish_part(GemmPart &g, std::vector<KUnit> &units, const std::vector<int32_t> &tap_off, hipStream_t stream,
                int siblings = 1, int k_floor = 0, int m_floor = 0) {
    // the kernel shape is fixed here because the packed weight layout depends on it
    g.cfg = GemmConfig();
    const bool equalize = k_floor > 0;
    const int k_len = g.k > k_floor ? g.k : k_floor;
    // a plain matrix: one tap at the pixel itself, unit stride, no padding (the tiled kernels then need no k-table)
    const bool plain_matrix = g.taps == 1 && g.proto.stride_h == 1 && g.proto.stride_w == 1 && g.proto.y_base == 0 && g.proto.x_base == 0 &&
                              g.proto.ho == g.proto.h && g.proto.wo == g.proto.w && g.vec == 16 && g.cin == g.proto.cin && !units.empty() &&
                              units[0].dy == 0 && units[0].dx == 0 && units[0].offset == 0;
    const bool ktab_fits = (size_t)(round_up(k_len > 0 ? k_len : 1, 256) / 16) * sizeof(KUnit) <= igemm_dma_ktab_limit();
    if (!equalize && !units.empty() && units[0].dy == 0 && units[0].dx == 0 &&
        igemm_thin_applies(g.taps, g.cin, g.proto.cin, units[0].offset, g.proto.y_base, g.proto.x_base, g.proto.m, g.n) &&
        // the one-tap kernel does not test its pixel against the image: every output pixel's tap must lie inside
        // (bottom / right padding of a 1x1 convolution, or a deconvolution phase enlarged by a negative tail padding,
        // go to the kernels that do)
        (g.proto.ho - 1) * g.proto.stride_h < g.proto.h && (g.proto.wo - 1) * g.proto.stride_w < g.proto.w) {
        g.cfg.id = GEMM_THIN;
        g.cfg.slab = 32;
    } else if (!equalize && !units.empty() && units[0].dy == 0 && units[0].dx == 0 && g.vec == 16 && g.k == g.cin &&
               gemm_skinny_applies(g.taps, g.cin, g.proto.cin, units[0].offset, g.proto.m, g.n) && g.proto.stride_h == 1 && g.proto.stride_w == 1 &&
               g.proto.y_base == 0 && g.proto.x_base == 0 && g.proto.h == g.proto.ho && g.proto.w == g.proto.wo && g.proto.out_sy == 1 &&
               g.proto.out_sx == 1 && g.proto.out_y0 == 0 && g.proto.out_x0 == 0 && g.proto.out_h == g.proto.ho && g.proto.out_w == g.proto.wo) {
        // a classifier head at batch 1 .. 64: the launch is the weights' one trip from memory
        g.cfg.id = GEMM_SKINNY;
        g.cfg.slab = 32;
    } else if (!equalize && g.cin == 3 && g.proto.cin == 3 && g.taps == 9 && g.k == 27 && units.size() == 27 && units[26].dy == 2 &&
               units[26].dx == 2 && units[12].dy == 1 && units[12].dx == 1 && units[0].offset == 0) {
        // three channels, 3x3 taps, dilation 1: the first layer of image networks
        g.cfg.id = GEMM_C3K3;
        g.cfg.slab = 32;
    } else if (int kh = 0, kw = 0; !equalize && g.cin >= 1 && g.cin <= 4 && g.taps > 1 && g.k == g.taps * g.cin && !units.empty() && units[0].offset == 0 &&
                                   units_are_rows(units, g.cin / g.vec, g.taps, kh, kw) && conv_rows_applies(g.cin, g.proto.cin, kh, kw) &&
                                   (long)g.proto.h * g.proto.w * g.cin >= 16) {
        // one to four input channels, a kernel row within 32 bytes: first layers on RGB(A) or grey images beyond 3x3 RGB
        g.cfg.id = GEMM_ROWS;
        g.cfg.slab = 32;
        g.proto.rows_kh = kh;
        g.proto.rows_kw = kw;
    } else if (!equalize && g.vec == 16 && g.taps == 9 && g.k == 9 * g.cin && units.size() == (size_t)g.k / 16 && g.proto.stride_h == 1 &&
               g.proto.stride_w == 1 && g.proto.out_sy == 1 && g.proto.out_sx == 1 && g.proto.out_y0 == 0 && g.proto.out_x0 == 0 &&
               g.proto.out_h == g.proto.ho && g.proto.out_w == g.proto.wo && units_are_3x3(units, g.cin / 16) &&
               conv3x3_patch_applies(g.cin, g.proto.cin, g.proto.wo, g.proto.ho) &&
               // (128 channels and a full round of 128 x 128 tiles or more: the implicit GEMM is the faster one, measured 15.0
               // against 20.6 us at 28 x 28 and 59.5 against 81.9 us at 56 x 56, batch 64, 128 output channels)
               !(g.cin >= 128 && (long)((g.proto.m + 127) / 128) * ((g.n + 127) / 128) >= 240)) {
        // 3x3 taps at dilation 1 and stride 1 over all input channels: the patch-in-LDS kernel
        g.cfg.id = GEMM_CONV3X3;
        g.cfg.slab = 32;
    } else if (g.vec == 16 && (ktab_fits || (plain_matrix && g.k % 256 == 0)))
        // (a reduction too long for its k-table to fit LDS still runs as a plain matrix of whole slabs: a fully
        // connected layer on 25088 inputs)
        g.cfg = igemm_dma_select(g.proto.m > m_floor ? g.proto.m : m_floor, g.n, g.k, siblings);  // (m_floor: the siblings' largest row count)
    bool must_slice = false;
    if (g.cfg.id == GEMM_STAGED && g.vec == 16 && !ktab_fits && siblings == 1 && g.n_period == 0) {
        // table-driven and too long for one k-table (a 7x7 convolution over 512 channels): the split-reduction tiles
        // with the reduction sliced, each slice under its own part of the table -- if few enough slices do it (below)
        g.cfg.id = GEMM_DMA_64x64_SPLITK;
        g.cfg.slab = 256;
        must_slice = true;
    }
    g.k_pad = g.cfg.id == GEMM_ROWS ? g.proto.rows_kh * 32 : round_up(k_len > 0 ? k_len : 1, g.cfg.slab);
    g.n_pad = round_up(g.n, igemm_n_tile(0, g.n, g.k));
    g.slices = 0;
    if (g.cfg.id == GEMM_DMA_64x64_SPLITK && siblings == 1 && g.n_period == 0) {
        // A launch of at most 64 tiles leaves three quarters of the CUs idle while each tile walks its whole reduction:
        // from 24 slabs on (6 KiB of reduction), up to four workgroups share a tile's reduction (at least 6 slabs each,
        // at most about 200 workgroups in all).  The second launch and the trip of the sums through memory cost about
        // 4 us, which shorter reductions do not win back (18 slabs, 3x3 on 512 channels at 7 x 7, batch 8: 12.0 us
        // either way; 45 slabs, 3x3 on 1280 channels at 10 x 10: 23.6 -> 14.1 us).
        const long tiles = (long)((g.proto.m + 63) / 64) * ((g.n + 63) / 64);
        const int slabs = g.k_pad / g.cfg.slab;
        // (a slice is table-driven: its part of the k-table has to fit)
        auto table_fits = [&](int n_slices) {
            return (size_t)(round_up(slabs, n_slices) / n_slices) * (g.cfg.slab / 16) * sizeof(KUnit) <= igemm_dma_ktab_limit();
        };
        int s = 4;
        if (must_slice) {
            // as few slices as fit their tables and a launch batch; the sums of all slices within 256 MiB
            s = 2;
            while (s <= GemmBatch::MAX && !table_fits(s)) ++s;
            if (s > GemmBatch::MAX || (size_t)s * g.proto.m * g.n_pad * 4 > ((size_t)256 << 20)) {
                s = 0;
                g.cfg = GemmConfig();  // the register-staged kernel after all
                g.k_pad = round_up(g.k > 0 ? g.k : 1, g.cfg.slab);
                g.n_pad = round_up(g.n, igemm_n_tile(0, g.n, g.k));
            }
        } else {
            while (s > 1 && (slabs < 6 * s || tiles * s > 208)) --s;
            if (!(tiles <= 64 && slabs >= 24 && s >= 2 && table_fits(s))) s = 0;
        }
        if (s >= 2) {
            g.slices = s;
            g.k_pad = round_up(g.k_pad, g.cfg.slab * s);
        }
    }
    KUnit pad;
    pad.offset = 0;
    pad.dy = INT16_MIN;
    pad.dx = 0;
    units.resize((size_t)g.k_pad / g.vec, pad);
    int rc;
    if ((rc = dev_alloc(&g.b, (size_t)g.n_pad * g.k_pad))) return rc;
    if ((rc = dev_alloc(&g.colsum, (size_t)g.n_pad))) return rc;
    if ((rc = dev_alloc(&g.folded, (size_t)g.n_pad))) return rc;
    if ((rc = dev_alloc(&g.ktab, units.size()))) return rc;
    if ((rc = dev_alloc(&g.tap_off, tap_off.size()))) return rc;
    if (g.slices && (rc = dev_alloc(&g.partial, (size_t)g.slices * g.proto.m * g.n_pad))) return rc;
    if (!g_dry_run) {
        EH_HIP(hipMemcpyAsync(g.ktab, units.data(), units.size() * sizeof(KUnit), hipMemcpyHostToDevice, stream));
        if (!tap_off.empty())
            EH_HIP(hipMemcpyAsync(g.tap_off, tap_off.data(), tap_off.size() * sizeof(int32_t), hipMemcpyHostToDevice, stream));
        // the host vectors die with the caller's frame: make sure the copies have left them
        EH_HIP(hipStreamSynchronize(stream));
    }
    g.proto.ktab = g.ktab;
    g.proto.a_offset = units.empty() ? 0 : units[0].offset;
    g.proto.k = g.k;
    g.proto.k_pad = g.k_pad;
    g.proto.vec = g.vec;
    g.proto.n = g.n;
    g.proto.cfg = g.cfg;
    g.proto.div_plane = make_fastdiv((uint32_t)(g.proto.ho * g.proto.wo));
    g.proto.div_wo = make_fastdiv((uint32_t)g.proto.wo);
    // a plain matrix: one tap at the pixel itself, unit stride, no padding, whole slabs
    // (a reduction that ends inside its last slab is handled by the kernel: the chunks past the end read a constant)
    g.proto.dense = plain_matrix ? 1 : 0;
    if (g.slices || equalize) g.proto.dense = 0;  // slices are cut out of the k-table; siblings of one launch all run table-driven
    return EH_OK;
}

int pack_part(GemmPart &g, const uint8_t *weight, bool w_signed, hipStream_t stream, int32_t off_block = 0) {
    PackProblem pp;
    pp.w = weight + g.w_base;
    pp.w_signed = w_signed ? 1 : 0;
    pp.bias = nullptr;
    pp.b = g.b;
    pp.colsum = g.colsum;
    pp.cfg = g.cfg;
    pp.n = g.n;
    pp.n_pad = g.n_pad;
    pp.cin = g.cin > 0 ? g.cin : 1;
    pp.taps = g.taps;
    pp.k = g.k;
    pp.k_pad = g.k_pad;
    pp.row_bytes = g.cfg.id == GEMM_ROWS ? g.proto.rows_kw * g.cin : 0;
    pp.cin_real = g.cin_real;
    pp.n_period = g.n_period;
    pp.period_step = g.period_step;
    pp.block_cin = g.block_cin;
    pp.block_n = g.block_n;
    pp.off_block = off_block;
    pp.so = g.so;
    pp.sc = g.sc;
    pp.tap_off = g.tap_off;
    return launch_pack_weights(pp, stream);
}

// Shared state of the three GEMM-shaped operators.
static int check_perchannel(const int32_t *multipliers, const int32_t *shifts, int32_t count) {
    for (int32_t i = 0; i < count; ++i)
        EH_REQUIRE(multipliers[i] >= 0 && shifts[i] >= -31 && shifts[i] <= 30, "per-channel multiplier/shift %d out of range", i);
    return EH_OK;
}

static bool all_pairs_fast(const int32_t *multipliers, const int32_t *shifts, int32_t count, int32_t max_shift = -1) {
    for (int32_t i = 0; i < count; ++i)
        if (!channel_pair_is_fast(multipliers[i], shifts[i], max_shift)) return false;
    return true;
}

// The per-channel arrays with `pad` entries behind them (kernels read whole channel blocks), written by one
// blocking copy each from a padded host image, once the stream's earlier work that may still read the arrays is
// done.
static int upload_padded_pairs(int32_t *d_mult, int32_t *d_shift, const int32_t *multipliers, const int32_t *shifts,
                               int32_t count, int32_t pad, hipStream_t stream) {
    std::vector<int32_t> image((size_t)count + pad, 0);
    EH_HIP(hipStreamSynchronize(stream));
    std::copy(multipliers, multipliers + count, image.begin());
    EH_HIP(hipMemcpy(d_mult, image.data(), image.size() * sizeof(int32_t), hipMemcpyHostToDevice));
    std::copy(shifts, shifts + count, image.begin());
    std::fill(image.begin() + count, image.end(), -2);  // the padding pairs stay inside the single-shift form's range
    EH_HIP(hipMemcpy(d_shift, image.data(), image.size() * sizeof(int32_t), hipMemcpyHostToDevice));
    return EH_OK;
}

struct GemmOp {
    std::vector<GemmPart> parts;
    int32_t *bias_copy = nullptr;  // the operator's own copy of the int32 bias
    int32_t cout = 0;
    eh_requant q{};
    bool folded_valid = false;
    // NCHW boundary: the kernels compute channels-last, so planar tensors pass
    // through these two staging images
    uint8_t *stage_in = nullptr, *stage_out = nullptr;
    uint8_t *fillbuf = nullptr;  // 16 x input zero point, 16 x 0x80: what out-of-image / padding chunks read
    int32_t layout = EH_NHWC;
    int32_t in_n = 0, in_c = 0, in_hw = 0, out_hw = 0;
    size_t in_bytes = 0;
    // Channel padding.  Channel counts (per group) that are no multiple of 16 would leave the byte-gathering kernel as
    // the only choice; instead the kernels then read a copy of the input in which every group's `pad_cg` channels are
    // followed by bytes holding the input zero point up to `pad_cg_to` channels, a multiple of 16.  Such a byte
    // contributes (zp_in - zp_in) * (w - zp_w) = 0 whatever weight it meets (the packed weights hold 0 there), so the
    // padded problem is the caller's problem exactly.
    int32_t pad_groups = 0, pad_cg = 0, pad_cg_to = 0;
    bool exact_channels = false;  // the caller asked for no padded copy
    // block-diagonal bundles of groups: the operator's copy of the weights and the zero point they were last packed with
    uint8_t *w_keep = nullptr;
    size_t w_keep_bytes = 0;
    int32_t packed_zp_w = INT32_MIN;
    uint8_t *stage_pad = nullptr;
    // int8 weights (value = byte as signed; zp_w is then an int8 zero point) and one multiplier / shift per
    // output channel instead of the requant's single pair
    bool has_bias = true;
    bool w_signed = false;
    bool io_signed = false;  // input and output tensors hold int8 values
    int32_t *pc_multiplier = nullptr, *pc_shift = nullptr;
    bool pc_fast = false;  // every channel's pair is inside the range of the kernels' per-channel single-shift form

    int zp_w_u8(const eh_requant &r) const { return r.zp_w + (w_signed ? 128 : 0); }  // zero point of the equivalent uint8 weights

    int set_perchannel(const int32_t *multipliers, const int32_t *shifts, int32_t count, hipStream_t stream) {
        if (multipliers == nullptr && shifts == nullptr) {
            EH_HIP(hipStreamSynchronize(stream));
            dev_free(pc_multiplier);
            dev_free(pc_shift);
            for (auto &g : parts) {
                dev_free(g.pc_multiplier_rep);
                dev_free(g.pc_shift_rep);
            }
            return EH_OK;
        }
        EH_REQUIRE(multipliers != nullptr && shifts != nullptr && count == cout, "per-channel arrays must hold %d entries (got %d)", cout, count);
        int rc = check_perchannel(multipliers, shifts, count);
        if (rc) return rc;
        // padded so that the kernels may read whole channel blocks
        if (!pc_multiplier && (rc = dev_alloc(&pc_multiplier, (size_t)cout + 512))) return rc;
        if (!pc_shift && (rc = dev_alloc(&pc_shift, (size_t)cout + 512))) return rc;
        pc_fast = all_pairs_fast(multipliers, shifts, cout, -2);  // the table form's rounding term needs rs >= 2
        if ((rc = upload_padded_pairs(pc_multiplier, pc_shift, multipliers, shifts, cout, 512, stream))) return rc;
        for (auto &g : parts) {
            if (g.n_period == 0) continue;
            std::vector<int32_t> m_rep((size_t)g.n), s_rep((size_t)g.n);
            for (int i = 0; i < g.n; ++i) {
                m_rep[i] = multipliers[g.bias_base + i % g.n_period];
                s_rep[i] = shifts[g.bias_base + i % g.n_period];
            }
            if (!g.pc_multiplier_rep && (rc = dev_alloc(&g.pc_multiplier_rep, (size_t)g.n + 512))) return rc;
            if (!g.pc_shift_rep && (rc = dev_alloc(&g.pc_shift_rep, (size_t)g.n + 512))) return rc;
            if ((rc = upload_padded_pairs(g.pc_multiplier_rep, g.pc_shift_rep, m_rep.data(), s_rep.data(), g.n, 512, stream))) return rc;
        }
        return EH_OK;
    }

    void release() {
        for (auto &g : parts) g.release();
        parts.clear();
        dev_free(bias_copy);
        dev_free(stage_in);
        dev_free(stage_out);
        dev_free(stage_pad);
        dev_free(w_keep);
        dev_free(fillbuf);
        dev_free(pc_multiplier);
        dev_free(pc_shift);
    }

    int set_weights(const void *weight, const void *bias, hipStream_t stream) {
        EH_REQUIRE(weight != nullptr, "weight pointer is null");
        if (!fillbuf) {
            int rc = dev_alloc(&fillbuf, 256);
            if (rc) return rc;
        }
        if (w_keep_bytes) {  // packed by refold(), which knows the zero point
            if (!w_keep) {
                int rc = dev_alloc(&w_keep, w_keep_bytes);
                if (rc) return rc;
            }
            EH_HIP(hipMemcpyAsync(w_keep, weight, w_keep_bytes, hipMemcpyDeviceToDevice, stream));
            packed_zp_w = INT32_MIN;
        } else {
            for (auto &g : parts) {
                int rc = pack_part(g, static_cast<const uint8_t *>(weight), w_signed, stream);
                if (rc) return rc;
            }
        }
        has_bias = bias != nullptr;  // no bias: the fold kernel takes zeros (no memset, so that a caller may capture this)
        if (bias) EH_HIP(hipMemcpyAsync(bias_copy, bias, (size_t)cout * sizeof(int32_t), hipMemcpyDeviceToDevice, stream));
        folded_valid = false;
        return EH_OK;
    }

    // `caller_q` as the caller states it; `q` keeps the uint8-equivalent input/output side
    int refold(const eh_requant &caller_q, hipStream_t stream) {
        const eh_requant nq = io_signed ? io_as_uint8(caller_q) : caller_q;
        if (folded_valid && nq.zp_in == q.zp_in && nq.zp_w == q.zp_w) {  // (w_signed and io_signed are fixed per plan)
            q = nq;
            return EH_OK;
        }
        if (w_keep_bytes && packed_zp_w != zp_w_u8(nq)) {
            EH_REQUIRE(w_keep != nullptr, "weights were never set");
            for (auto &g : parts) {
                int rc = pack_part(g, w_keep, w_signed, stream, zp_w_u8(nq) - 128);
                if (rc) return rc;
            }
            packed_zp_w = zp_w_u8(nq);
        }
        for (auto &g : parts) {
            int rc = launch_fold_bias(has_bias ? bias_copy + g.bias_base : nullptr, g.colsum, g.folded, g.n, g.n_pad, g.k, nq.zp_in, zp_w_u8(nq),
                                      fillbuf, io_signed ? 0x80 : 0, stream, g.n_period);
            if (rc) return rc;
        }
        q = nq;
        folded_valid = true;
        return EH_OK;
    }

    // the one-tap kernel, the split-reduction epilogue of the tiled kernel and the kernel for few rows can add a residual tensor
    bool fuses_add() const {
        bool fuse = layout == EH_NHWC && !io_signed && !parts.empty();
        for (auto &g : parts) fuse = fuse && (g.cfg.id == GEMM_THIN || g.cfg.id == GEMM_DMA_64x64_SPLITK || g.cfg.id == GEMM_SKINNY);
        return fuse;
    }

    // residual != null: output = add(residual, result) with `radd`; `fused` tells whether the kernels did it
    // bytes of the two channels-last staging images of a planar plan (each with the slack the kernels' wide loads need)
    size_t stage_in_bytes() const { return ((size_t)in_n * in_c * in_hw + 256 + 255) / 256 * 256; }
    size_t stage_out_bytes() const { return ((size_t)in_n * cout * out_hw + 256 + 255) / 256 * 256; }
    size_t stage_pad_bytes() const { return ((size_t)in_n * in_hw * pad_groups * pad_cg_to + 256 + 255) / 256 * 256; }
    // what a run that brings its own staging memory needs: the planar plan's two images, then the padded input
    size_t staging_bytes() const { return (layout == EH_NCHW ? stage_in_bytes() + stage_out_bytes() : 0) + (pad_cg_to ? stage_pad_bytes() : 0); }
    int alloc_staging() {
        int rc = EH_OK;
        if (layout == EH_NCHW) {
            if ((rc = dev_alloc(&stage_in, stage_in_bytes()))) return rc;
            if ((rc = dev_alloc(&stage_out, stage_out_bytes()))) return rc;
        }
        if (pad_cg_to) rc = dev_alloc(&stage_pad, stage_pad_bytes());
        return rc;
    }
    static constexpr int kInlineParts = 8;  // a run over at most this many parts allocates no host memory

    // One part's kernel argument for channels-last tensors `in` / `out`, with the quantization parameters refold() left in `q`
    GemmProblem problem(const GemmPart &g, const uint8_t *in, uint8_t *out, const uint8_t *residual, const AddDev *radd) const {
        GemmProblem p = g.proto;
        p.a = in;
        p.b = g.b;
        p.bias = g.folded;
        p.fillbuf = fillbuf;
        p.out = out + g.bias_base;
        p.zw = zp_w_u8(q) - 128;
        p.out_xor = io_signed ? 0x80808080u : 0u;
        p.a_xor = 0x80808080u ^ p.out_xor;
        p.fill = ((uint32_t)q.zp_in * 0x01010101u) ^ p.out_xor;
        p.rq = make_requant_dev(q);
        p.residual = residual ? residual + g.bias_base : nullptr;
        if (residual) p.radd = *radd;
        if (pc_multiplier) {
            p.rq.pc_multiplier = g.n_period ? g.pc_multiplier_rep : pc_multiplier + g.bias_base;
            p.rq.pc_shift = g.n_period ? g.pc_shift_rep : pc_shift + g.bias_base;
            // every kernel but the register-staged one has the single-shift form per channel (the first-layer
            // kernel for fewer than 32 channels ignores the flag)
            const bool has_form = g.cfg.id != GEMM_STAGED;
            p.rq.fast = (pc_fast && has_form) ? channel_fast_mode(q) : 0;
        }
        return p;
    }

    // staging != null: the plan uses [staging, staging + staging_bytes()) instead of its own images
    int run(const void *input, void *output, const eh_requant *nq, hipStream_t stream, const uint8_t *residual = nullptr,
            const AddDev *radd = nullptr, bool *fused = nullptr, uint8_t *staging = nullptr) {
        EH_REQUIRE(input != nullptr && output != nullptr, "input/output pointer is null");
        int rc = check_requant(nq, w_signed, io_signed);
        if (rc) return rc;
        const bool fuse = residual != nullptr && fuses_add();
        if (fused) *fused = fuse;
        if ((rc = refold(*nq, stream))) return rc;
        const uint8_t *in = static_cast<const uint8_t *>(input);
        uint8_t *out = static_cast<uint8_t *>(output);
        uint8_t *const st_in = staging ? staging : stage_in, *const st_out = staging ? staging + stage_in_bytes() : stage_out;
        if (layout == EH_NCHW) {
            if ((rc = launch_nchw2nhwc(in, st_in, in_n, in_c, in_hw, stream))) return rc;
            in = st_in;
            out = st_out;
        }
        if (pad_cg_to) {
            uint8_t *const st_pad = staging ? staging + (layout == EH_NCHW ? stage_in_bytes() + stage_out_bytes() : 0) : stage_pad;
            // (q holds the uint8-equivalent input zero point after refold(); int8 tensors store it minus 128)
            if ((rc = launch_pad_channels(in, st_pad, (int64_t)in_n * in_hw, pad_groups, pad_cg, pad_cg_to,
                                          (uint32_t)(q.zp_in & 0xFF) ^ (io_signed ? 0x80u : 0u), stream)))
                return rc;
            in = st_pad;
        }
        GemmProblem inline_problems[kInlineParts];
        std::vector<GemmProblem> many;
        size_t launches = 0;
        for (auto &g : parts) launches += g.slices ? (size_t)g.slices : 1;
        if (launches > (size_t)kInlineParts) many.resize(launches);
        GemmProblem *const problems = many.empty() ? inline_problems : many.data();
        int filled = 0;
        for (auto &g : parts) {
            EH_REQUIRE((reinterpret_cast<uintptr_t>(in) & (uintptr_t)(g.vec - 1)) == 0,
                       "input pointer is not aligned to %d bytes", g.vec);
            const GemmProblem whole = problem(g, in, out, fuse ? residual : nullptr, radd);
            if (g.slices == 0) {
                problems[filled++] = whole;
                continue;
            }
            // equal runs of slabs, one problem each: its part of the k-table and of every packed row block
            const int slabs = g.k_pad / g.cfg.slab, run = slabs / g.slices;
            for (int s = 0; s < g.slices; ++s) {
                GemmProblem slice = whole;
                slice.ktab = whole.ktab + (size_t)s * run * (g.cfg.slab / 16);
                slice.b = whole.b + (size_t)s * run * 1024;
                slice.b_slabs = slabs;
                slice.k_pad = run * g.cfg.slab;
                slice.k = slice.k_pad;
                slice.partial = g.partial + (size_t)s * whole.m * g.n_pad;
                slice.partial_ld = g.n_pad;
                slice.residual = nullptr;
                problems[filled++] = slice;
            }
        }
        if ((rc = launch_igemm_batch(problems, filled, stream))) return rc;
        for (auto &g : parts)
            if (g.slices && (rc = launch_splitk_finish(problem(g, in, out, fuse ? residual : nullptr, radd), g.partial, g.n_pad, g.slices, stream))) return rc;
        if (layout == EH_NCHW) {
            if ((rc = launch_nhwc2nchw(st_out, static_cast<uint8_t *>(output), in_n, cout, out_hw, stream))) return rc;
        }
        return EH_OK;
    }
};

int check_desc_common(const eh_conv_desc *d, bool negative_tail_padding = false) {
    EH_REQUIRE(d != nullptr, "descriptor is null");
    EH_REQUIRE(d->n >= 0 && d->c > 0 && d->h > 0 && d->w > 0 && d->cout > 0, "bad tensor extents n=%d c=%d h=%d w=%d cout=%d",
               d->n, d->c, d->h, d->w, d->cout);
    EH_REQUIRE(d->kh > 0 && d->kw > 0 && d->stride_h > 0 && d->stride_w > 0, "bad kernel/stride");
    // a transposed convolution may state a negative bottom / right padding: it only enlarges the output
    // (cl_optimized_impls/CLDeconvolutionQuantized.cpp:254-256 uses the top / left values alone)
    EH_REQUIRE(d->pad_t >= 0 && d->pad_l >= 0 && (negative_tail_padding || (d->pad_b >= 0 && d->pad_r >= 0)), "negative padding");
    EH_REQUIRE(d->layout == EH_NCHW || d->layout == EH_NHWC, "unknown layout %d", d->layout);
    EH_REQUIRE((int64_t)d->n * d->c * d->h * d->w < (1ll << 31), "input larger than 2 GiB is not supported");
    EH_REQUIRE(d->h < 32000 && d->w < 32000, "spatial extent too large");
    return EH_OK;
}

}  // namespace
}  // namespace eh

using namespace eh;

struct eh_conv_plan {
    GemmOp op;
    eh_conv_desc d;
};
struct eh_fc_plan {
    GemmOp op;
    int32_t m, k, n;
};
struct eh_deconv_plan {
    GemmOp op;
    eh_conv_desc d;
};
struct eh_dwconv_plan {
    eh_conv_desc d;
    int32_t ho = 0, wo = 0, cout = 0, taps = 0;
    uint8_t *w_copy = nullptr;
    int32_t *bias_copy = nullptr;
    int32_t *w_pair = nullptr;
    int32_t *bias_folded = nullptr;
    eh_requant q{};
    bool packed_valid = false;
    bool w_signed = false, io_signed = false, has_bias = true;
    int32_t *pc_multiplier = nullptr, *pc_shift = nullptr;  // [cout + 4] once per-channel pairs are set
    bool pc_fast = false;  // every pair is inside the single-shift form's range
    // 3x3 channels-last plans: the 8-bit dot product form of the weights, usable while every w - zp_w fits int8
    int32_t *w_trip = nullptr, *bias_trip = nullptr;
    int32_t *w_fold = nullptr, *bias_fold = nullptr;  // the unsigned form of the same plans, for weights of any range
    bool fold_valid = false;
    // 5x5 / 7x7 channels-last plans: the unsigned form with two words per kernel column
    int32_t *w_foldk = nullptr, *bias_foldk = nullptr;
    bool foldk_valid = false;
    bool range_known = false;   // w_lo / w_hi hold the extremes of the weight bytes (in the caller's own domain)
    int32_t w_lo = 0, w_hi = 0;
    bool trip_valid = false;    // w_trip / bias_trip match the current zero points
    // Staging.  `d` describes what the kernels run: channels-last tensors with depth multiplier 1.  A caller's depth
    // multiplier m > 1 (channels-last) is met by a copy of the input with every channel m times in a row, so that
    // output channel j reads channel j of the copy; a caller's planar tensors (multiplier 1) by the two transpositions
    // the convolution plans use.  Both only where the output channels are a multiple of 4 (the four-channel kernels).
    int32_t rep_c = 0, rep_dm = 0;  // the caller's channel count and depth multiplier when the input is replicated
    // ... and output channels that are no multiple of 4 (channels-last) by rounding them up: the copy of the input ends
    // every pixel with repeats of its last channel, the weights of the extra channels are zero, and the result is
    // computed into an image of the padded width, from which the caller's channels are copied out.
    int32_t cout_caller = 0;        // `cout` counts the padded channels; this is what the caller's tensors hold
    bool planar = false;            // the caller's tensors are NCHW
    uint8_t *stage_in = nullptr, *stage_out = nullptr;
};

extern "C" {

int eh_requant_apply(const eh_requant *q, const int32_t *acc, uint8_t *out, int64_t count, int32_t form,
                                int32_t *single_shift) {
    int rc = check_requant(q);
    if (rc) return rc;
    EH_REQUIRE(count >= 0 && (count == 0 || (acc && out)), "requant_apply: null array");
    EH_REQUIRE(form >= 0 && form <= 4, "requant_apply: form %d", form);
    const RequantDev r = make_requant_dev(*q);
    if (form == 2 || form == 3) {  // the per-channel single-shift forms, with the requant's pair as the channel's
        EH_REQUIRE(channel_pair_is_fast(q->multiplier, q->shift, form == 3 ? -2 : -1) && channel_fast_mode(*q) != 0,
                   "requant_apply: multiplier %d, shift %d, zero point %d are outside form %d", q->multiplier, q->shift, q->zp_out, form);
        const int mode = channel_fast_mode(*q), rs = -q->shift;
        if (single_shift) *single_shift = 1;
        for (int64_t i = 0; i < count; ++i) {
            uint32_t v;
            if (form == 2)
                v = mode == 2 ? requant_u8_channel_fast<2>(acc[i], q->multiplier, q->shift, r) : requant_u8_channel_fast<1>(acc[i], q->multiplier, q->shift, r);
            else
                v = mode == 2 ? requant_u8_channel_table<2>(acc[i], q->multiplier, rs - 1, channel_table_pos_hi(q->zp_out, rs), r)
                              : requant_u8_channel_table<1>(acc[i], q->multiplier, rs - 1, channel_table_pos_hi(q->zp_out, rs), r);
            out[i] = (uint8_t)v;
        }
        return EH_OK;
    }
    if (form == 4) {  // four at a time, a row term of up to +-4000 (varying with the group) held back from the accumulators
        EH_REQUIRE(r.fast != 0, "requant_apply: multiplier %d, shift %d, zero point %d are outside form 4", q->multiplier, q->shift, q->zp_out);
        if (single_shift) *single_shift = 1;
        for (int64_t i = 0; i < count; i += 4) {
            const int32_t extra = (int32_t)(((uint64_t)(i + 1) * 2654435761ull >> 13) % 8001) - 4000;
            int32_t x[4];
            for (int t = 0; t < 4; ++t) x[t] = (int32_t)((uint32_t)acc[i + t < count ? i + t : count - 1] - (uint32_t)extra);
            const uint32_t w = r.fast == 2 ? requant4_fast<2>(x[0], x[1], x[2], x[3], extra, r) : requant4_fast<1>(x[0], x[1], x[2], x[3], extra, r);
            for (int t = 0; t < 4 && i + t < count; ++t) out[i + t] = (uint8_t)(w >> (8 * t));
        }
        return EH_OK;
    }
    const bool fast = form == 0 && r.fast;
    if (single_shift) *single_shift = fast ? 1 : 0;
    for (int64_t i = 0; i < count; ++i)
        out[i] = (uint8_t)(!fast ? requant_u8(acc[i], r) : r.fast == 2 ? requant_u8_fast_relu(acc[i], r) : requant_u8_fast(acc[i], r));
    return EH_OK;
}


// ------------------------------------------------------------ host arithmetic

void eh_quantize_multiplier(double real_multiplier, int32_t *quantized_multiplier, int32_t *shift) {
    if (real_multiplier == 0.) {
        *quantized_multiplier = 0;
        *shift = 0;
        return;
    }
    int exponent = 0;
    const double significand = frexp(real_multiplier, &exponent);
    int64_t fixed = (int64_t)round(significand * 2147483648.0);
    if (fixed == 2147483648ll) {
        fixed /= 2;
        ++exponent;
    }
    *quantized_multiplier = (int32_t)fixed;
    *shift = exponent;
}

int eh_conv_multiplier(float input_scale, float filter_scale, float bias_scale, float output_scale, double *multiplier) {
    const double product = (double)input_scale * (double)filter_scale;
    const double bs = (double)bias_scale;
    if (!(fabs(product - bs) <= 1e-6 * (product < bs ? product : bs))) return EH_FAILURE;
    if (!(product >= 0)) return EH_FAILURE;
    *multiplier = product / (double)output_scale;
    return EH_OK;
}

static void act_range(int activation, float scale, int32_t zero_point, int32_t lo, int32_t hi, int32_t *act_min,
                      int32_t *act_max) {
    auto quantize = [scale, zero_point](float f) { return zero_point + (int32_t)round((double)(f / scale)); };
    if (activation == EH_ACT_RELU) {
        lo = quantize(0.0f) > lo ? quantize(0.0f) : lo;
    } else if (activation == EH_ACT_RELU6) {
        lo = quantize(0.0f) > lo ? quantize(0.0f) : lo;
        hi = quantize(6.0f) < hi ? quantize(6.0f) : hi;
    } else if (activation == EH_ACT_RELU1) {
        lo = quantize(-1.0f) > lo ? quantize(-1.0f) : lo;
        hi = quantize(1.0f) < hi ? quantize(1.0f) : hi;
    }
    *act_min = lo;
    *act_max = hi;
}

void eh_act_range_u8(int activation, float scale, int32_t zero_point, int32_t *act_min, int32_t *act_max) {
    act_range(activation, scale, zero_point, 0, 255, act_min, act_max);
}

void eh_act_range_s8(int activation, float scale, int32_t zero_point, int32_t *act_min, int32_t *act_max) {
    act_range(activation, scale, zero_point, -128, 127, act_min, act_max);
}

void eh_make_requant_s8(float input_scale, int32_t input_zp, float filter_scale, int32_t filter_zp, float bias_scale,
                        float output_scale, int32_t output_zp, int activation, int activation_enabled, eh_requant *out) {
    eh_make_requant(input_scale, input_zp, filter_scale, filter_zp, bias_scale, output_scale, output_zp, activation, 0, out);
    out->act_min = -128;
    out->act_max = 127;
    if (activation_enabled) eh_act_range_s8(activation, output_scale, output_zp, &out->act_min, &out->act_max);
}

void eh_make_requant(float input_scale, int32_t input_zp, float filter_scale, int32_t filter_zp, float bias_scale,
                     float output_scale, int32_t output_zp, int activation, int activation_enabled, eh_requant *out) {
    double m = 0.0;  // stays 0 when the bias scale check fails, as in the reference's callers
    (void)eh_conv_multiplier(input_scale, filter_scale, bias_scale, output_scale, &m);
    eh_quantize_multiplier(m, &out->multiplier, &out->shift);
    if (out->shift < -31) {
        // |acc * M| < 2^31 * 2^-32 rounds to 0 for every int32 accumulator
        out->multiplier = 0;
        out->shift = 0;
    }
    out->zp_in = input_zp;
    out->zp_w = filter_zp;
    out->zp_out = output_zp;
    if (activation_enabled) {
        eh_act_range_u8(activation, output_scale, output_zp, &out->act_min, &out->act_max);
    } else {
        out->act_min = 0;
        out->act_max = 255;
    }
}

void eh_make_requant_perchannel(float input_scale, int32_t input_zp, const float *filter_scales, int32_t channels,
                                float output_scale, int32_t output_zp, int activation, int activation_enabled, eh_requant *out,
                                int32_t *multipliers, int32_t *shifts) {
    out->zp_in = input_zp;
    out->zp_w = 0;
    out->zp_out = output_zp;
    out->multiplier = 0;
    out->shift = 0;
    for (int32_t i = 0; i < channels; ++i) {
        // the bias scale handed to the check is input_scale * scales[i] by construction, so it always passes
        double m = 0.0;
        (void)eh_conv_multiplier(input_scale, filter_scales[i], input_scale * filter_scales[i], output_scale, &m);
        eh_quantize_multiplier(m, &multipliers[i], &shifts[i]);
    }
    out->act_min = 0;
    out->act_max = 255;
    if (activation_enabled) eh_act_range_u8(activation, output_scale, output_zp, &out->act_min, &out->act_max);
}

int32_t eh_conv_out_dim(int32_t in, int32_t pad_a, int32_t pad_b, int32_t kernel, int32_t dilation, int32_t stride) {
    return (in + pad_a + pad_b - (dilation * (kernel - 1) + 1) + stride) / stride;
}

int32_t eh_deconv_out_dim(int32_t in, int32_t pad_a, int32_t pad_b, int32_t kernel, int32_t stride) {
    return in * stride + kernel - stride - pad_a - pad_b;
}

// ------------------------------------------------------------ runtime

const char *eh_last_error(void) { return g_error; }

int eh_init(int device) {
    int count = 0;
    EH_HIP(hipGetDeviceCount(&count));
    EH_REQUIRE(device >= 0 && device < count, "device %d not present (%d visible)", device, count);
    EH_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    EH_HIP(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        set_error("device %d is %s; this library carries gfx950 code only", device, prop.gcnArchName);
        return EH_FAILURE;
    }
    int rc = conv3x3_patch_prepare();  // per-device kernel attributes, set here so that no launch has to
    if (rc) return rc;
    uint8_t *unused = nullptr;
    return static_scratch(&unused);  // this device's address of the static scratch, asked for while the device is current
}

int eh_device_name(char *dst, size_t cap) {
    EH_REQUIRE(dst != nullptr && cap > 0, "bad destination");
    int dev = 0;
    EH_HIP(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    EH_HIP(hipGetDeviceProperties(&prop, dev));
    snprintf(dst, cap, "%s (%s, %d CUs)", prop.name, prop.gcnArchName, prop.multiProcessorCount);
    return EH_OK;
}

int eh_malloc(void **ptr, size_t bytes) {
    EH_REQUIRE(ptr != nullptr, "null result pointer");
    *ptr = nullptr;
    const size_t padded = (bytes + 255) / 256 * 256 + 256;
    EH_HIP(hipMalloc(ptr, padded));
    // The fill is queued on the null stream and hipMemset may return before it has run; the streams this library
    // hands out do not synchronize with the null stream, so the caller's first write on such a stream could otherwise
    // be overtaken by the zeros.  Wait for the fill.
    hipError_t e = hipMemset(*ptr, 0, padded);
    if (e == hipSuccess) e = hipStreamSynchronize(nullptr);
    if (e != hipSuccess) {
        (void)hipFree(*ptr);
        *ptr = nullptr;
        return hip_fail(e, "hipMemset");
    }
    return EH_OK;
}

int eh_free(void *ptr) {
    if (ptr) EH_HIP(hipFree(ptr));
    return EH_OK;
}

int eh_memset(void *ptr, int value, size_t bytes, void *stream) {
    if (bytes) EH_HIP(hipMemsetAsync(ptr, value, bytes, as_stream(stream)));
    return EH_OK;
}

int eh_h2d(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes) EH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(stream)));
    return EH_OK;
}

int eh_d2h(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes) EH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, as_stream(stream)));
    return EH_OK;
}

int eh_d2d(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes) EH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
    return EH_OK;
}

int eh_stream_sync(void *stream) {
    EH_HIP(hipStreamSynchronize(as_stream(stream)));
    return EH_OK;
}

int eh_stream_create(void **stream) {
    EH_REQUIRE(stream != nullptr, "null result pointer");
    hipStream_t s;
    EH_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *stream = s;
    return EH_OK;
}

int eh_stream_destroy(void *stream) {
    if (stream) EH_HIP(hipStreamDestroy(as_stream(stream)));
    return EH_OK;
}

int eh_graph_begin(void *stream) {
    EH_REQUIRE(stream != nullptr, "graph capture needs a stream made by eh_stream_create");
    EH_HIP(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeThreadLocal));
    return EH_OK;
}

int eh_graph_end(void *stream, void **graph) {
    EH_REQUIRE(stream != nullptr && graph != nullptr, "null argument");
    *graph = nullptr;
    hipGraph_t g = nullptr;
    EH_HIP(hipStreamEndCapture(as_stream(stream), &g));
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (e != hipSuccess) return hip_fail(e, "hipGraphInstantiate");
    *graph = exec;
    return EH_OK;
}

int eh_graph_launch(void *graph, void *stream) {
    EH_REQUIRE(graph != nullptr, "null graph");
    EH_HIP(hipGraphLaunch(reinterpret_cast<hipGraphExec_t>(graph), as_stream(stream)));
    return EH_OK;
}

int eh_graph_destroy(void *graph) {
    if (graph) EH_HIP(hipGraphExecDestroy(reinterpret_cast<hipGraphExec_t>(graph)));
    return EH_OK;
}

int eh_event_create(void **event) {
    EH_REQUIRE(event != nullptr, "null result pointer");
    hipEvent_t e;
    EH_HIP(hipEventCreate(&e));
    *event = e;
    return EH_OK;
}

int eh_event_record(void *event, void *stream) {
    EH_HIP(hipEventRecord(reinterpret_cast<hipEvent_t>(event), as_stream(stream)));
    return EH_OK;
}

int eh_stream_wait_event(void *stream, void *event) {
    EH_REQUIRE(event != nullptr, "null event");
    EH_HIP(hipStreamWaitEvent(as_stream(stream), reinterpret_cast<hipEvent_t>(event), 0));
    return EH_OK;
}

int eh_event_elapsed_ms(void *start, void *stop, float *ms) {
    EH_HIP(hipEventSynchronize(reinterpret_cast<hipEvent_t>(stop)));
    EH_HIP(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(start), reinterpret_cast<hipEvent_t>(stop)));
    return EH_OK;
}

int eh_event_destroy(void *event) {
    if (event) EH_HIP(hipEventDestroy(reinterpret_cast<hipEvent_t>(event)));
    return EH_OK;
}

// ------------------------------------------------------------ layout

int eh_transpose_u8_nchw2nhwc(const void *src, void *dst, int32_t n, int32_t c, int32_t h, int32_t w, void *stream) {
    EH_REQUIRE(n >= 0 && c >= 0 && h >= 0 && w >= 0, "negative extent");
    if ((int64_t)n * c * h * w == 0) return EH_OK;
    EH_REQUIRE(src != nullptr && dst != nullptr && src != dst, "bad pointers");
    EH_REQUIRE((int64_t)h * w < (1ll << 31), "plane too large");
    return launch_nchw2nhwc(static_cast<const uint8_t *>(src), static_cast<uint8_t *>(dst), n, c, h * w, as_stream(stream));
}

int eh_transpose_u8_nhwc2nchw(const void *src, void *dst, int32_t n, int32_t c, int32_t h, int32_t w, void *stream) {
    EH_REQUIRE(n >= 0 && c >= 0 && h >= 0 && w >= 0, "negative extent");
    if ((int64_t)n * c * h * w == 0) return EH_OK;
    EH_REQUIRE(src != nullptr && dst != nullptr && src != dst, "bad pointers");
    EH_REQUIRE((int64_t)h * w < (1ll << 31), "plane too large");
    return launch_nhwc2nchw(static_cast<const uint8_t *>(src), static_cast<uint8_t *>(dst), n, c, h * w, as_stream(stream));
}

// Whether a plan just built on the caller's channel count should be built again on padded channels: some part fell to
// the byte-gathering kernel.  Sets the padding up and drops the parts if so.
static bool wants_channel_padding(GemmOp &op, int groups, int channels_per_group) {
    if (op.exact_channels || op.pad_cg_to != 0 || (channels_per_group & 15) == 0) return false;
    bool staged = false;
    for (const GemmPart &g : op.parts) staged = staged || (g.cfg.id == GEMM_STAGED && g.k > 0);
    if (!staged) return false;
    const int64_t padded = (int64_t)op.in_n * op.in_hw * groups * round_up(channels_per_group, 16);
    if (padded >= (1ll << 31)) return false;
    for (auto &g : op.parts) g.release();
    op.parts.clear();
    dev_free(op.bias_copy);
    op.pad_groups = groups;
    op.pad_cg = channels_per_group;
    op.pad_cg_to = round_up(channels_per_group, 16);
    return true;
}

// ------------------------------------------------------------ convolution

static int conv_plan_build(eh_conv_plan *pl, const eh_conv_desc *d, hipStream_t stream) {
    GemmOp &op = pl->op;
    const int G = d->groups;
    int cig = d->c / G, cog = d->cout / G;
    const int ho = eh_conv_out_dim(d->h, d->pad_t, d->pad_b, d->kh, d->dil_h, d->stride_h);
    const int wo = eh_conv_out_dim(d->w, d->pad_l, d->pad_r, d->kw, d->dil_w, d->stride_w);
    EH_REQUIRE(ho > 0 && wo > 0, "convolution output is empty (%d x %d)", ho, wo);
    EH_REQUIRE((int64_t)d->n * ho * wo < (1ll << 31), "too many output pixels");
    EH_REQUIRE((int64_t)d->n * ho * wo * d->cout < (1ll << 31) * 2, "output larger than 4 GiB is not supported");
    op.cout = d->cout;
    op.layout = d->layout;
    op.in_n = d->n;
    op.in_c = d->c;
    op.in_hw = d->h * d->w;
    op.out_hw = ho * wo;
    int rc;
    if ((rc = dev_alloc(&op.bias_copy, (size_t)d->cout))) return rc;
    const int taps = d->kh * d->kw;
    // built on the caller's channel count first; when that leaves a group to the byte-gathering kernel, built again on
    // channels padded to a multiple of 16
    const int cig_real = cig;
    const bool padded = op.pad_cg_to != 0;
    if (padded) cig = op.pad_cg_to;
    const int pixel_c = padded ? G * cig : d->c;
    // Groups of fewer than 16 channels each (ResNeXt-style 3x3 layers): `bundle` neighbouring groups run as one
    // block-diagonal problem over their 16 .. 64 adjacent channels, read in 16-byte units straight from the tensor,
    // instead of one small problem per group on a padded copy.
    int bundle = 1;
    if (G > 1 && !padded && !op.exact_channels && (cig & 15) != 0)
        for (int b = G; b >= 2 && bundle == 1; --b)
            if (G % b == 0 && b * cig <= 64 && ((b * cig) & 15) == 0) bundle = b;
    op.w_keep_bytes = bundle > 1 ? (size_t)d->cout * cig * taps : 0;
    const int parts_n = G / bundle;
    cig *= bundle;
    cog *= bundle;
    op.parts.resize(parts_n);
    for (int g = 0; g < parts_n; ++g) {
        GemmPart &part = op.parts[g];
        part.n = cog;
        part.cin = cig;
        part.cin_real = padded ? cig_real : 0;
        part.block_cin = bundle > 1 ? cig / bundle : 0;
        part.block_n = bundle > 1 ? cog / bundle : 0;
        part.taps = taps;
        part.k = taps * cig;
        part.vec = pick_vec(cig, pixel_c);
        part.bias_base = g * cog;
        if (d->weight_layout == EH_W_OIHW) {
            part.so = (int64_t)cig_real * taps;
            part.sc = taps;
        } else {
            part.so = (int64_t)taps * cig_real;
            part.sc = 1;
        }
        part.w_base = (int64_t)g * cog * part.so;
        std::vector<int32_t> tap_off(taps);
        for (int t = 0; t < taps; ++t) tap_off[t] = d->weight_layout == EH_W_OIHW ? t : t * cig_real;
        std::vector<KUnit> units;
        for (int k = 0; k < part.k; k += part.vec) {
            const int t = k / cig, c = k - t * cig;
            const int ky = t / d->kw, kx = t - ky * d->kw;
            KUnit u;
            u.dy = (int16_t)(ky * d->dil_h);
            u.dx = (int16_t)(kx * d->dil_w);
            u.offset = (u.dy * d->w + u.dx) * pixel_c + g * cig + c;
            units.push_back(u);
        }
        GemmProblem &p = part.proto;
        p.m = d->n * ho * wo;
        p.h = d->h;
        p.w = d->w;
        p.cin = pixel_c;
        p.ho = ho;
        p.wo = wo;
        p.stride_h = d->stride_h;
        p.stride_w = d->stride_w;
        p.y_base = -d->pad_t;
        p.x_base = -d->pad_l;
        p.out_h = ho;
        p.out_w = wo;
        p.out_sy = 1;
        p.out_sx = 1;
        p.out_y0 = 0;
        p.out_x0 = 0;
        p.ldc = d->cout;
        if ((rc = finish_part(part, units, tap_off, stream, std::min(parts_n, (int)GemmBatch::MAX)))) return rc;
    }
    if (wants_channel_padding(op, G, cig_real)) return conv_plan_build(pl, d, stream);
    return op.alloc_staging();
}

// `desc` with the two flag bits taken out, checked
static int conv_desc_checked(const eh_conv_desc *desc, eh_conv_desc *plain) {
    EH_REQUIRE(desc != nullptr, "descriptor is null");
    *plain = *desc;
    plain->weight_layout &= ~EH_W_SIGNED;
    plain->layout &= ~(EH_IO_SIGNED | EH_EXACT_CHANNELS);
    desc = plain;
    int rc = check_desc_common(desc);
    if (rc) return rc;
    EH_REQUIRE(desc->dil_h > 0 && desc->dil_w > 0, "bad dilation");
    EH_REQUIRE(desc->groups > 0 && desc->c % desc->groups == 0 && desc->cout % desc->groups == 0,
               "groups %d do not divide channels (%d, %d)", desc->groups, desc->c, desc->cout);
    EH_REQUIRE(desc->weight_layout == EH_W_OIHW || desc->weight_layout == EH_W_OHWI, "bad convolution weight layout %d",
               desc->weight_layout);
    EH_REQUIRE(desc->kh * desc->dil_h < 32000 && desc->kw * desc->dil_w < 32000, "kernel extent too large");
    EH_REQUIRE((int64_t)desc->c * desc->kh * desc->kw <= EH_MAX_REDUCTION,
               "reductions over %lld terms (all groups) are not supported (at most %d)", (long long)desc->c * desc->kh * desc->kw, EH_MAX_REDUCTION);
    return EH_OK;
}

static int report_kernels(const GemmOp &op, int32_t *kernel_ids, int32_t cap) {
    for (size_t i = 0; i < op.parts.size() && (int32_t)i < cap; ++i) kernel_ids[i] = op.parts[i].cfg.id;
    return (int)op.parts.size();
}

int eh_conv2d_u8_kernels(const eh_conv_desc *desc, int32_t *kernel_ids, int32_t cap) {
    EH_REQUIRE(kernel_ids != nullptr || cap == 0, "null result array");
    eh_conv_desc plain;
    int rc = conv_desc_checked(desc, &plain);
    if (rc) return rc;
    if (plain.n == 0) return 0;
    eh_conv_plan pl;
    pl.op.exact_channels = (desc->layout & EH_EXACT_CHANNELS) != 0;
    g_dry_run = true;
    rc = conv_plan_build(&pl, &plain, nullptr);
    g_dry_run = false;
    return rc ? rc : report_kernels(pl.op, kernel_ids, cap);
}

int eh_conv2d_u8_plan(eh_conv_plan **plan, const eh_conv_desc *desc, const void *weight, const void *bias,
                      const eh_requant *q, void *stream) {
    EH_REQUIRE(plan != nullptr, "null plan pointer");
    *plan = nullptr;
    EH_REQUIRE(desc != nullptr, "descriptor is null");
    const bool w_signed = (desc->weight_layout & EH_W_SIGNED) != 0, io_signed = (desc->layout & EH_IO_SIGNED) != 0;
    const bool exact_channels = (desc->layout & EH_EXACT_CHANNELS) != 0;
    eh_conv_desc plain;
    int rc = conv_desc_checked(desc, &plain);
    if (rc) return rc;
    desc = &plain;
    if ((rc = check_requant(q, w_signed, io_signed))) return rc;
    eh_conv_plan *pl = new (std::nothrow) eh_conv_plan();
    EH_REQUIRE(pl != nullptr, "out of host memory");
    pl->d = *desc;
    pl->op.w_signed = w_signed;
    pl->op.io_signed = io_signed;
    pl->op.exact_channels = exact_channels;
    if (desc->n > 0) {
        rc = conv_plan_build(pl, desc, as_stream(stream));
        if (!rc) rc = pl->op.set_weights(weight, bias, as_stream(stream));
        if (!rc) rc = pl->op.refold(*q, as_stream(stream));
        if (rc) {
            pl->op.release();
            delete pl;
            return rc;
        }
    }
    *plan = pl;
    return EH_OK;
}

int eh_conv2d_u8_set_perchannel(eh_conv_plan *plan, const int32_t *multipliers, const int32_t *shifts, int32_t count,
                                void *stream) {
    EH_REQUIRE(plan != nullptr, "null plan");
    if (plan->d.n == 0) return EH_OK;
    return plan->op.set_perchannel(multipliers, shifts, count, as_stream(stream));
}

int eh_conv2d_u8_repack(eh_conv_plan *plan, const void *weight, const void *bias, const eh_requant *q, void *stream) {
    EH_REQUIRE(plan != nullptr, "null plan");
    int rc = check_requant(q, plan->op.w_signed, plan->op.io_signed);
    if (rc) return rc;
    if (plan->d.n == 0) return EH_OK;
    if ((rc = plan->op.set_weights(weight, bias, as_stream(stream)))) return rc;
    return plan->op.refold(*q, as_stream(stream));
}

int eh_conv2d_u8_run(eh_conv_plan *plan, const void *input, void *output, const eh_requant *q, void *stream) {
    EH_REQUIRE(plan != nullptr, "null plan");
    if (plan->d.n == 0) return check_requant(q, plan->op.w_signed, plan->op.io_signed);  // zero-size early-out, as CLConvolution::execute does
    return plan->op.run(input, output, q, as_stream(stream));
}

int eh_conv2d_u8_run_static(eh_conv_plan *plan, const void *input, void *output, const eh_requant *q, void *stream) {
    EH_REQUIRE(plan != nullptr, "null plan");
    if (plan->d.n == 0) return check_requant(q, plan->op.w_signed, plan->op.io_signed);
    const GemmOp &op = plan->op;
    size_t problems = 0;  // (beyond the inline array a run would allocate host memory)
    for (const GemmPart &g : op.parts) problems += g.slices ? (size_t)g.slices : 1;
    EH_REQUIRE(problems <= (size_t)GemmOp::kInlineParts, "run_static: the plan runs as %zu problems (groups, slices), at most %d are supported",
               problems, GemmOp::kInlineParts);
    uint8_t *staging = nullptr;
    if (const size_t need = op.staging_bytes(); need != 0) {
        EH_REQUIRE(need <= (size_t)EH_STATIC_SCRATCH_BYTES,
                   "run_static: the staging images of this plan (channels-last, channel-padded) take %zu bytes, the static scratch holds %zu", need,
                   (size_t)EH_STATIC_SCRATCH_BYTES);
        int rc = static_scratch(&staging);
        if (rc) return rc;
    }
    // every staging byte a kernel reads was written earlier in the same call, so nothing has to be cleared
    return plan->op.run(input, output, q, as_stream(stream), nullptr, nullptr, nullptr, staging);
}

int eh_conv2d_u8_run_add(eh_conv_plan *plan, const void *input, const void *residual, void *output, const eh_requant *q,
                         const eh_add_requant *aq, void *stream) {
    EH_REQUIRE(plan != nullptr, "null plan");
    EH_REQUIRE(!plan->op.io_signed, "run_add: int8 tensors are not offered (the reference's int8 add is a float kernel)");
    int rc = check_add_requant(aq);
    if (rc) return rc;
    if (plan->d.n == 0) return check_requant(q, plan->op.w_signed, plan->op.io_signed);
    EH_REQUIRE(residual != nullptr, "run_add: residual pointer is null");
    const AddDev radd = make_add_dev(*aq);
    bool fused = false;
    if ((rc = plan->op.run(input, output, q, as_stream(stream), static_cast<const uint8_t *>(residual), &radd, &fused))) return rc;
    if (fused) return EH_OK;
    // kernels without the fused epilogue: the convolution's own result, then the add in place
    const eh_conv_desc &d = plan->d;
    const int64_t count = (int64_t)d.n * d.cout * eh_conv_out_dim(d.h, d.pad_t, d.pad_b, d.kh, d.dil_h, d.stride_h) *
                          eh_conv_out_dim(d.w, d.pad_l, d.pad_r, d.kw, d.dil_w, d.stride_w);
    return launch_add_u8(static_cast<const uint8_t *>(residual), static_cast<const uint8_t *>(output),
                         static_cast<uint8_t *>(output), count, radd, as_stream(stream));
}

int eh_conv2d_u8_fuses_add(const eh_conv_plan *plan) { return plan != nullptr && plan->op.fuses_add() ? 1 : 0; }

int eh_conv2d_u8_destroy(eh_conv_plan *plan) {
    if (plan) {
        plan->op.release();
        delete plan;
    }
    return EH_OK;
}

// ------------------------------------------------------------ fully connected

int eh_fc_u8_plan(eh_fc_plan **plan, int32_t m, int32_t k, int32_t n, const void *weight, const void *bias,
                  const eh_requant *q, void *stream) {
    return eh_fc_q8_plan(plan, m, k, n, 0, weight, bias, q, stream);
}

int eh_fc_q8_plan(eh_fc_plan **plan, int32_t m, int32_t k, int32_t n, int32_t flags, const void *weight, const void *bias,
                  const eh_requant *q, void *stream) {
    EH_REQUIRE(plan != nullptr, "null plan pointer");
    *plan = nullptr;
    EH_REQUIRE(m >= 0 && k > 0 && n > 0, "bad extents m=%d k=%d n=%d", m, k, n);
    EH_REQUIRE((int64_t)m * k < (1ll << 31), "input larger than 2 GiB is not supported");
    EH_REQUIRE(k <= EH_MAX_REDUCTION, "a reduction over %d terms is not supported (at most %d)", k, EH_MAX_REDUCTION);
    EH_REQUIRE((flags & ~(EH_W_SIGNED | EH_IO_SIGNED | EH_EXACT_CHANNELS)) == 0, "unknown flags 0x%x", flags);
    const bool w_signed = (flags & EH_W_SIGNED) != 0, io_signed = (flags & EH_IO_SIGNED) != 0;
    int rc = check_requant(q, w_signed, io_signed);
    if (rc) return rc;
    eh_fc_plan *pl = new (std::nothrow) eh_fc_plan();
    EH_REQUIRE(pl != nullptr, "out of host memory");
    pl->m = m;
    pl->k = k;
    pl->n = n;
    GemmOp &op = pl->op;
    op.w_signed = w_signed;
    op.io_signed = io_signed;
    op.exact_channels = (flags & EH_EXACT_CHANNELS) != 0;
    op.cout = n;
    op.layout = EH_NHWC;
    op.in_n = m;
    op.in_c = k;
    op.in_hw = 1;
    op.out_hw = 1;
    hipStream_t s = as_stream(stream);
    // (a second pass on a row length padded to a multiple of 16 when the first leaves the byte-gathering kernel)
    const int k_real = k;
    for (int pass = 0; pass < 2 && !rc; ++pass) {
        if (pass == 1) {
            if (!wants_channel_padding(op, 1, k_real)) break;
            k = op.pad_cg_to;
        }
        rc = dev_alloc(&op.bias_copy, (size_t)n);
        if (rc) break;
        op.parts.resize(1);
        GemmPart &part = op.parts[0];
        part.n = n;
        part.cin = k;
        part.cin_real = pass == 1 ? k_real : 0;
        part.taps = 1;
        part.k = k;
        part.vec = pick_vec(k, k);
        part.so = k_real;
        part.sc = 1;
        std::vector<int32_t> tap_off(1, 0);
        std::vector<KUnit> units;
        for (int kk = 0; kk < k; kk += part.vec) {
            KUnit u;
            u.dy = 0;
            u.dx = 0;
            u.offset = kk;
            units.push_back(u);
        }
        GemmProblem &p = part.proto;
        p.m = m;
        p.h = 1;
        p.w = 1;
        p.cin = k;
        p.ho = 1;
        p.wo = 1;
        p.stride_h = 1;
        p.stride_w = 1;
        p.y_base = 0;
        p.x_base = 0;
        p.out_h = 1;
        p.out_w = 1;
        p.out_sy = 1;
        p.out_sx = 1;
        p.out_y0 = 0;
        p.out_x0 = 0;
        p.ldc = n;
        rc = finish_part(part, units, tap_off, s);
    }
    if (!rc) rc = op.alloc_staging();
    if (!rc) rc = op.set_weights(weight, bias, s);
    if (!rc) rc = op.refold(*q, s);
    if (rc) {
        op.release();
        delete pl;
        return rc;
    }
    *plan = pl;
    return EH_OK;
}

int eh_fc_u8_repack(eh_fc_plan *plan, const void *weight, const void *bias, const eh_requant *q, void *stream) {
    EH_REQUIRE(plan != nullptr, "null plan");
    int rc = check_requant(q, plan->op.w_signed, plan->op.io_signed);
    if (rc) return rc;
    if ((rc = plan->op.set_weights(weight, bias, as_stream(stream)))) return rc;
    return plan->op.refold(*q, as_stream(stream));
}

int eh_fc_u8_run(eh_fc_plan *plan, const void *input, void *output, const eh_requant *q, void *stream) {
    EH_REQUIRE(plan != nullptr, "null plan");
    if (plan->m == 0) return check_requant(q, plan->op.w_signed, plan->op.io_signed);
    return plan->op.run(input, output, q, as_stream(stream));
}

int eh_fc_u8_destroy(eh_fc_plan *plan) {
    if (plan) {
        plan->op.release();
        delete plan;
    }
    return EH_OK;
}

// ------------------------------------------------------------ deconvolution
// A transposed convolution with stride s splits into s_h * s_w independent
// stride-1 convolutions, one per output phase (oy + pad_t) mod s_h,
// (ox + pad_l) mod s_w: phase (py, px) uses the taps ky = py + s_h*ty,
// kx = px + s_w*tx and writes every s-th output pixel.  Each phase is one
// implicit GEMM with the epilogue fused, so the reference's int32 col buffer
// (N*Hi*Wi*Cout*kh*kw*4 bytes, CLDeconvolutionQuantized.cpp:99-103) never exists.

static int deconv_plan_build(eh_deconv_plan *pl, const eh_conv_desc *d, hipStream_t stream) {
    GemmOp &op = pl->op;
    const int G = d->groups, cog = d->cout / G;
    int cig = d->c / G;
    const int oh = eh_deconv_out_dim(d->h, d->pad_t, d->pad_b, d->kh, d->stride_h);
    const int ow = eh_deconv_out_dim(d->w, d->pad_l, d->pad_r, d->kw, d->stride_w);
    EH_REQUIRE(oh > 0 && ow > 0, "deconvolution output is empty (%d x %d)", oh, ow);
    EH_REQUIRE((int64_t)d->n * oh * ow * d->cout < (1ll << 31) * 2, "output larger than 4 GiB is not supported");
    op.cout = d->cout;
    op.layout = d->layout;
    op.in_n = d->n;
    op.in_c = d->c;
    op.in_hw = d->h * d->w;
    op.out_hw = oh * ow;
    int rc;
    if ((rc = dev_alloc(&op.bias_copy, (size_t)d->cout))) return rc;
    // (built a second time on channels padded to a multiple of 16 when a phase is left to the byte-gathering kernel)
    const int cig_real = cig;
    const bool padded = op.pad_cg_to != 0;
    if (padded) cig = op.pad_cg_to;
    const int pixel_c = padded ? G * cig : d->c;
    const int sh = d->stride_h, sw = d->stride_w;
    // Output columns ox0, ox0 + 1, ... whose phases read the same input columns (their kernel columns px, px + 1, ...
    // differ, their taps' positions do not) and cover equally many positions go out as ONE problem whose columns are
    // (kernel column, output channel): a row of the problem then writes neighbouring output pixels, count * cout
    // contiguous bytes, and the launches shrink by that count.  Needs one group (a pixel holds the problem's channels
    // alone) and more than one tap (the one-tap kernel has its own batching) or an output channel count that is no
    // multiple of 16 (a phase alone would store rows of that many bytes at unaligned addresses).
    struct XPhase {
        int px, ox0, wo_p, ntx, bx;
    };
    // A kernel that is no multiple of the stride (3x3 at stride 2) gives phases with 4, 2, 2 and 1 taps.  Padding every
    // phase's reduction to the longest and choosing the tile shape for the largest phase puts them into one launch
    // instead of one launch each (the phases' pixel counts may differ by a row or a column: every problem of a launch
    // tests rows against its own count); accepted up to twice the multiply-adds.
    int k_floor = 0, m_floor = 0;
    if (G == 1 && (cig & 15) == 0 && (d->kh % sh != 0 || d->kw % sw != 0) && sh * sw <= GemmBatch::MAX) {
        long taps_max = 0, taps_sum = 0;
        int phases = 0;
        for (int py = 0; py < sh; ++py)
            for (int px = 0; px < sw; ++px) {
                const int oy0 = ((py - d->pad_t) % sh + sh) % sh, ox0 = ((px - d->pad_l) % sw + sw) % sw;
                if (oy0 >= oh || ox0 >= ow) continue;
                const long m_p = (long)((oh - oy0 + sh - 1) / sh) * ((ow - ox0 + sw - 1) / sw);
                const long taps_p = (long)(py < d->kh ? (d->kh - py + sh - 1) / sh : 0) * (px < d->kw ? (d->kw - px + sw - 1) / sw : 0);
                m_floor = (int)std::max((long)m_floor, (long)d->n * m_p);
                taps_max = std::max(taps_max, taps_p);
                taps_sum += taps_p;
                ++phases;
            }
        if (phases >= 2 && taps_max * phases <= 2 * taps_sum && taps_max * phases > taps_sum) k_floor = (int)taps_max * cig;
    }
    for (int g = 0; g < G; ++g)
        for (int py = 0; py < sh; ++py) {
            const int oy0 = ((py - d->pad_t) % sh + sh) % sh;
            if (oy0 >= oh) continue;
            const int ho_p = (oh - oy0 + sh - 1) / sh;
            const int nty = py < d->kh ? (d->kh - py + sh - 1) / sh : 0;
            const int by = (oy0 + d->pad_t - py) / sh;
            std::vector<XPhase> xs;
            for (int px = 0; px < sw; ++px) {
                XPhase x;
                x.px = px;
                x.ox0 = ((px - d->pad_l) % sw + sw) % sw;
                if (x.ox0 >= ow) continue;
                x.wo_p = (ow - x.ox0 + sw - 1) / sw;
                x.ntx = px < d->kw ? (d->kw - px + sw - 1) / sw : 0;
                x.bx = (x.ox0 + d->pad_l - px) / sw;
                xs.push_back(x);
            }
            std::sort(xs.begin(), xs.end(), [](const XPhase &a, const XPhase &b) { return a.ox0 < b.ox0; });
            for (size_t first = 0; first < xs.size();) {
                const XPhase &x0 = xs[first];
                size_t last = first + 1;
                while (G == 1 && (nty * x0.ntx > 1 || (cog & 15) != 0) && last < xs.size() && xs[last].ox0 == xs[last - 1].ox0 + 1 &&
                       xs[last].px == xs[last - 1].px + 1 && xs[last].bx == x0.bx && xs[last].wo_p == x0.wo_p && xs[last].ntx == x0.ntx)
                    ++last;
                const int count = (int)(last - first);
                first = last;
                const int px = x0.px, ox0 = x0.ox0, wo_p = x0.wo_p, ntx = x0.ntx, bx = x0.bx;
                op.parts.emplace_back();
                GemmPart &part = op.parts.back();
                part.n = cog * count;
                part.cin = cig;
                part.cin_real = padded ? cig_real : 0;
                part.taps = nty * ntx;
                part.k = part.taps * cig;
                part.vec = pick_vec(cig, pixel_c);
                part.bias_base = g * cog;
                std::vector<int32_t> tap_off(part.taps > 0 ? part.taps : 0);
                if (d->weight_layout == EH_W_IOHW) {
                    part.so = (int64_t)d->kh * d->kw;
                    part.sc = (int64_t)cog * d->kh * d->kw;
                    part.w_base = (int64_t)g * cig_real * cog * d->kh * d->kw;
                    part.period_step = 1;
                } else {  // OHWI, groups == 1
                    part.so = (int64_t)d->kh * d->kw * d->c;
                    part.sc = 1;
                    part.w_base = 0;
                    part.period_step = d->c;
                }
                part.n_period = count > 1 ? cog : 0;
                for (int ty = 0; ty < nty; ++ty)
                    for (int tx = 0; tx < ntx; ++tx) {
                        const int ky = py + sh * ty, kx = px + sw * tx;
                        tap_off[ty * ntx + tx] = d->weight_layout == EH_W_IOHW ? ky * d->kw + kx : (ky * d->kw + kx) * d->c;
                    }
                std::vector<KUnit> units;
                for (int k = 0; k < part.k; k += part.vec) {
                    const int t = k / cig, c = k - t * cig;
                    const int ty = t / ntx, tx = t - ty * ntx;
                    KUnit u;
                    u.dy = (int16_t)(by - ty);
                    u.dx = (int16_t)(bx - tx);
                    u.offset = (u.dy * d->w + u.dx) * pixel_c + g * cig + c;
                    units.push_back(u);
                }
                GemmProblem &p = part.proto;
                p.m = d->n * ho_p * wo_p;
                p.h = d->h;
                p.w = d->w;
                p.cin = pixel_c;
                p.ho = ho_p;
                p.wo = wo_p;
                p.stride_h = 1;
                p.stride_w = 1;
                p.y_base = 0;
                p.x_base = 0;
                p.out_h = oh;
                p.out_w = ow;
                p.out_sy = sh;
                p.out_sx = sw;
                p.out_y0 = oy0;
                p.out_x0 = ox0;
                p.ldc = d->cout;
                // phases (and groups) of equal shape share launches: choose the tile shape for the joint tile count
                const int siblings = (k_floor > 0 || (d->kh % sh == 0 && d->kw % sw == 0)) ? std::min(G * sh * sw / count, (int)GemmBatch::MAX) : 1;
                if ((rc = finish_part(part, units, tap_off, stream, siblings, k_floor, k_floor ? m_floor : 0))) return rc;
            }
        }
    if (wants_channel_padding(op, G, cig_real)) return deconv_plan_build(pl, d, stream);
    return op.alloc_staging();
}

static int deconv_desc_checked(const eh_conv_desc *desc, eh_conv_desc *plain) {
    EH_REQUIRE(desc != nullptr, "descriptor is null");
    *plain = *desc;
    plain->weight_layout &= ~EH_W_SIGNED;
    plain->layout &= ~(EH_IO_SIGNED | EH_EXACT_CHANNELS);
    desc = plain;
    int rc = check_desc_common(desc, true);
    if (rc) return rc;
    EH_REQUIRE(desc->groups > 0 && desc->c % desc->groups == 0 && desc->cout % desc->groups == 0,
               "groups %d do not divide channels (%d, %d)", desc->groups, desc->c, desc->cout);
    EH_REQUIRE(desc->weight_layout == EH_W_IOHW || desc->weight_layout == EH_W_OHWI, "bad deconvolution weight layout %d",
               desc->weight_layout);
    EH_REQUIRE(desc->weight_layout == EH_W_IOHW || desc->groups == 1, "OHWI weights support groups == 1 only");
    EH_REQUIRE((int64_t)desc->groups * desc->stride_h * desc->stride_w <= 65536, "%lld output phases (groups x strides) are not supported (at most 65536)",
               (long long)desc->groups * desc->stride_h * desc->stride_w);
    EH_REQUIRE((int64_t)desc->c * desc->kh * desc->kw <= EH_MAX_REDUCTION,
               "reductions over %lld terms (all groups) are not supported (at most %d)", (long long)desc->c * desc->kh * desc->kw, EH_MAX_REDUCTION);
    return EH_OK;
}

int eh_deconv2d_u8_kernels(const eh_conv_desc *desc, int32_t *kernel_ids, int32_t cap) {
    EH_REQUIRE(kernel_ids != nullptr || cap == 0, "null result array");
    eh_conv_desc plain;
    int rc = deconv_desc_checked(desc, &plain);
    if (rc) return rc;
    if (plain.n == 0) return 0;
    eh_deconv_plan pl;
    pl.op.exact_channels = (desc->layout & EH_EXACT_CHANNELS) != 0;
    g_dry_run = true;
    rc = deconv_plan_build(&pl, &plain, nullptr);
    g_dry_run = false;
    return rc ? rc : report_kernels(pl.op, kernel_ids, cap);
}

int eh_deconv2d_u8_plan(eh_deconv_plan **plan, const eh_conv_desc *desc, const void *weight, const void *bias,
                        const eh_requant *q, void *stream) {
    EH_REQUIRE(plan != nullptr, "null plan pointer");
    *plan = nullptr;
    EH_REQUIRE(desc != nullptr, "descriptor is null");
    const bool w_signed = (desc->weight_layout & EH_W_SIGNED) != 0, io_signed = (desc->layout & EH_IO_SIGNED) != 0;
    const bool exact_channels = (desc->layout & EH_EXACT_CHANNELS) != 0;
    eh_conv_desc plain;
    int rc = deconv_desc_checked(desc, &plain);
    if (rc) return rc;
    desc = &plain;
    if ((rc = check_requant(q, w_signed, io_signed))) return rc;
    eh_deconv_plan *pl = new (std::nothrow) eh_deconv_plan();
    EH_REQUIRE(pl != nullptr, "out of host memory");
    pl->d = *desc;
    pl->op.w_signed = w_signed;
    pl->op.io_signed = io_signed;
    pl->op.exact_channels = exact_channels;
    if (desc->n > 0) {
        rc = deconv_plan_build(pl, desc, as_stream(stream));
        if (!rc) rc = pl->op.set_weights(weight, bias, as_stream(stream));
        if (!rc) rc = pl->op.refold(*q, as_stream(stream));
        if (rc) {
            pl->op.release();
            delete pl;
            return rc;
        }
    }
    *plan = pl;
    return EH_OK;
}

int eh_deconv2d_u8_set_perchannel(eh_deconv_plan *plan, const int32_t *multipliers, const int32_t *shifts, int32_t count,
                                  void *stream) {
    EH_REQUIRE(plan != nullptr, "null plan");
    if (plan->d.n == 0) return EH_OK;
    return plan->op.set_perchannel(multipliers, shifts, count, as_stream(stream));
}

int eh_deconv2d_u8_repack(eh_deconv_plan *plan, const void *weight, const void *bias, const eh_requant *q, void *stream) {
    EH_REQUIRE(plan != nullptr, "null plan");
    int rc = check_requant(q, plan->op.w_signed, plan->op.io_signed);
    if (rc) return rc;
    if (plan->d.n == 0) return EH_OK;
    if ((rc = plan->op.set_weights(weight, bias, as_stream(stream)))) return rc;
    return plan->op.refold(*q, as_stream(stream));
}

int eh_deconv2d_u8_run(eh_deconv_plan *plan, const void *input, void *output, const eh_requant *q, void *stream) {
    EH_REQUIRE(plan != nullptr, "null plan");
    if (plan->d.n == 0) return check_requant(q, plan->op.w_signed, plan->op.io_signed);
    return plan->op.run(input, output, q, as_stream(stream));
}

int eh_deconv2d_u8_destroy(eh_deconv_plan *plan) {
    if (plan) {
        plan->op.release();
        delete plan;
    }
    return EH_OK;
}

// ------------------------------------------------------------ depthwise

static void dw_release(eh_dwconv_plan *pl) {
    dev_free(pl->w_copy);
    dev_free(pl->bias_copy);
    dev_free(pl->w_pair);
    dev_free(pl->bias_folded);
    dev_free(pl->pc_multiplier);
    dev_free(pl->pc_shift);
    dev_free(pl->w_trip);
    dev_free(pl->bias_trip);
    dev_free(pl->w_fold);
    dev_free(pl->bias_fold);
    dev_free(pl->w_foldk);
    dev_free(pl->bias_foldk);
    dev_free(pl->stage_in);
    dev_free(pl->stage_out);
}

static int dw_set_weights(eh_dwconv_plan *pl, const void *weight, const void *bias, hipStream_t stream) {
    EH_REQUIRE(weight != nullptr, "weight pointer is null");
    if (pl->d.weight_layout == EH_W_OHWI) {  // [taps][cout] -> [cout][taps]
        int rc = launch_nhwc2nchw(static_cast<const uint8_t *>(weight), pl->w_copy, 1, pl->cout_caller, pl->taps, stream);
        if (rc) return rc;
    } else {
        EH_HIP(hipMemcpyAsync(pl->w_copy, weight, (size_t)pl->cout_caller * pl->taps, hipMemcpyDeviceToDevice, stream));
    }
    pl->has_bias = bias != nullptr;
    if (bias) EH_HIP(hipMemcpyAsync(pl->bias_copy, bias, (size_t)pl->cout_caller * sizeof(int32_t), hipMemcpyDeviceToDevice, stream));
    pl->packed_valid = false;
    pl->range_known = false;  // the plan call looks at the bytes once; weights replaced later keep the 16-bit form
    pl->trip_valid = false;
    return EH_OK;
}

static int dw_refold(eh_dwconv_plan *pl, const eh_requant &caller_q, hipStream_t stream) {
    const eh_requant q = pl->io_signed ? io_as_uint8(caller_q) : caller_q;  // pl->q: the uint8-equivalent input/output side
    if (!(pl->packed_valid && q.zp_in == pl->q.zp_in && q.zp_w == pl->q.zp_w)) {
        int rc = launch_dw_pack(pl->w_copy, pl->has_bias ? pl->bias_copy : nullptr, pl->w_pair, pl->bias_folded, pl->cout, pl->taps, q.zp_in,
                                q.zp_w, pl->w_signed ? 1 : 0, stream);
        if (rc) return rc;
        pl->trip_valid = false;
        if (pl->w_trip && pl->range_known && pl->w_lo - q.zp_w >= -128 && pl->w_hi - q.zp_w <= 127) {
            rc = launch_dw_pack_trip(pl->w_copy, pl->has_bias ? pl->bias_copy : nullptr, pl->w_trip, pl->bias_trip, pl->cout, q.zp_in,
                                     q.zp_w, pl->w_signed ? 1 : 0, stream);
            if (rc) return rc;
            pl->trip_valid = true;
        }
        pl->fold_valid = false;
        if (pl->w_fold && !pl->trip_valid) {
            rc = launch_dw_pack_fold(pl->w_copy, pl->has_bias ? pl->bias_copy : nullptr, pl->w_fold, pl->bias_fold, pl->cout, q.zp_in,
                                     q.zp_w + (pl->w_signed ? 128 : 0), pl->w_signed ? 1 : 0, stream);
            if (rc) return rc;
            pl->fold_valid = true;
        }
        pl->foldk_valid = false;
        if (pl->w_foldk) {
            rc = launch_dw_pack_foldk(pl->w_copy, pl->has_bias ? pl->bias_copy : nullptr, pl->w_foldk, pl->bias_foldk, pl->cout, pl->d.kh, q.zp_in,
                                      q.zp_w + (pl->w_signed ? 128 : 0), pl->w_signed ? 1 : 0, stream);
            if (rc) return rc;
            pl->foldk_valid = true;
        }
        pl->packed_valid = true;
    }
    pl->q = q;
    return EH_OK;
}

int eh_dwconv2d_u8_plan(eh_dwconv_plan **plan, const eh_conv_desc *desc, const void *weight, const void *bias,
                        const eh_requant *q, void *stream) {
    EH_REQUIRE(plan != nullptr, "null plan pointer");
    *plan = nullptr;
    EH_REQUIRE(desc != nullptr, "descriptor is null");
    const bool w_signed = (desc->weight_layout & EH_W_SIGNED) != 0, io_signed = (desc->layout & EH_IO_SIGNED) != 0;
    const bool no_staging = (desc->layout & EH_EXACT_CHANNELS) != 0;
    eh_conv_desc plain = *desc;
    plain.weight_layout &= ~EH_W_SIGNED;
    plain.layout &= ~(EH_IO_SIGNED | EH_EXACT_CHANNELS);
    desc = &plain;
    int rc = check_desc_common(desc);
    if (rc) return rc;
    if ((rc = check_requant(q, w_signed, io_signed))) return rc;
    EH_REQUIRE(desc->dil_h > 0 && desc->dil_w > 0, "bad dilation");
    EH_REQUIRE(desc->depth_multiplier > 0, "bad depth multiplier %d", desc->depth_multiplier);
    EH_REQUIRE(desc->cout == desc->c * desc->depth_multiplier, "depthwise cout %d != c %d * depth multiplier %d", desc->cout,
               desc->c, desc->depth_multiplier);
    EH_REQUIRE(desc->weight_layout == EH_W_OIHW || desc->weight_layout == EH_W_OHWI,
               "depthwise weights are [C*dm][1][kh][kw] (OIHW) or [1][kh][kw][C*dm] (OHWI)");
    eh_dwconv_plan *pl = new (std::nothrow) eh_dwconv_plan();
    EH_REQUIRE(pl != nullptr, "out of host memory");
    pl->d = *desc;
    pl->cout_caller = desc->cout;
    if (!no_staging && desc->n > 0) {
        const int32_t cout4 = (desc->cout + 3) & ~3;
        if (desc->layout == EH_NHWC && (desc->depth_multiplier > 1 || cout4 != desc->cout) &&
            (int64_t)desc->n * desc->h * desc->w * cout4 < (1ll << 31)) {
            pl->rep_c = desc->c;
            pl->rep_dm = desc->depth_multiplier;
            pl->d.c = cout4;
            pl->d.cout = cout4;
            pl->d.depth_multiplier = 1;
        } else if (desc->layout == EH_NCHW && desc->depth_multiplier == 1 && cout4 == desc->cout) {
            pl->planar = true;
            pl->d.layout = EH_NHWC;
        }
    }
    desc = &pl->d;
    pl->w_signed = w_signed;
    pl->io_signed = io_signed;
    pl->ho = eh_conv_out_dim(desc->h, desc->pad_t, desc->pad_b, desc->kh, desc->dil_h, desc->stride_h);
    pl->wo = eh_conv_out_dim(desc->w, desc->pad_l, desc->pad_r, desc->kw, desc->dil_w, desc->stride_w);
    pl->cout = desc->cout;
    pl->taps = desc->kh * desc->kw;
    if (pl->ho <= 0 || pl->wo <= 0) {
        delete pl;
        set_error("depthwise output is empty");
        return EH_INVALID_PARAMS;
    }
    hipStream_t s = as_stream(stream);
    rc = dev_alloc(&pl->w_copy, (size_t)pl->cout * pl->taps);
    if (!rc && (pl->rep_dm || pl->planar)) rc = dev_alloc(&pl->stage_in, (size_t)desc->n * desc->h * desc->w * pl->cout + 256);
    if (!rc && (pl->planar || pl->cout != pl->cout_caller)) rc = dev_alloc(&pl->stage_out, (size_t)desc->n * pl->ho * pl->wo * pl->cout + 256);
    if (!rc) rc = dev_alloc(&pl->bias_copy, (size_t)pl->cout);
    if (!rc && pl->cout != pl->cout_caller && !g_dry_run) {  // the extra channels: zero weights, zero bias
        EH_HIP(hipMemsetAsync(pl->w_copy, 0, (size_t)pl->cout * pl->taps, s));
        EH_HIP(hipMemsetAsync(pl->bias_copy, 0, (size_t)pl->cout * sizeof(int32_t), s));
    }
    if (!rc) rc = dev_alloc(&pl->w_pair, (size_t)((pl->taps + 1) / 2) * pl->cout);
    if (!rc) rc = dev_alloc(&pl->bias_folded, (size_t)pl->cout + 4);
    const bool tile_form = pl->d.layout == EH_NHWC && pl->d.kh == 3 && pl->d.kw == 3 && pl->d.depth_multiplier == 1;
    if (!rc && tile_form) {
        rc = dev_alloc(&pl->w_trip, (size_t)3 * pl->cout);
        if (!rc) rc = dev_alloc(&pl->bias_trip, (size_t)pl->cout + 4);
        if (!rc) rc = dev_alloc(&pl->w_fold, (size_t)3 * pl->cout);
        if (!rc) rc = dev_alloc(&pl->bias_fold, (size_t)pl->cout + 4);
    }
    const bool tile_form_k = pl->d.layout == EH_NHWC && pl->d.kh == pl->d.kw && (pl->d.kh == 5 || pl->d.kh == 7) && pl->d.depth_multiplier == 1 &&
                             pl->d.dil_h == 1 && pl->d.dil_w == 1;
    if (!rc && tile_form_k) {
        rc = dev_alloc(&pl->w_foldk, (size_t)pl->d.kw * 2 * pl->cout);
        if (!rc) rc = dev_alloc(&pl->bias_foldk, (size_t)pl->cout + 4);
    }
    if (!rc) rc = dw_set_weights(pl, weight, bias, s);
    if (!rc && tile_form && pl->cout > 0) {
        // the extremes of the weight bytes decide, per zero point, whether the 8-bit dot product form applies
        std::vector<uint8_t> host((size_t)pl->cout_caller * 9);
        hipError_t e = hipMemcpyAsync(host.data(), pl->w_copy, host.size(), hipMemcpyDeviceToHost, s);
        if (e == hipSuccess) e = hipStreamSynchronize(s);
        if (e != hipSuccess) {
            rc = hip_fail(e, "depthwise: weight download");
        } else {
            int lo = 255, hi = -128;
            for (uint8_t b : host) {
                const int v = pl->w_signed ? (int)(int8_t)b : (int)b;
                lo = v < lo ? v : lo;
                hi = v > hi ? v : hi;
            }
            pl->w_lo = lo;
            pl->w_hi = hi;
            pl->range_known = true;
        }
    }
    if (!rc) rc = dw_refold(pl, *q, s);
    if (rc) {
        dw_release(pl);
        delete pl;
        return rc;
    }
    *plan = pl;
    return EH_OK;
}

int eh_dwconv2d_u8_set_perchannel(eh_dwconv_plan *plan, const int32_t *multipliers, const int32_t *shifts, int32_t count,
                                  void *stream) {
    EH_REQUIRE(plan != nullptr, "null plan");
    if (multipliers == nullptr || shifts == nullptr) {
        EH_REQUIRE(multipliers == nullptr && shifts == nullptr, "per-channel: one of the two arrays is null");
        EH_HIP(hipStreamSynchronize(as_stream(stream)));  // a queued run may still read the arrays
        dev_free(plan->pc_multiplier);
        dev_free(plan->pc_shift);
        plan->pc_multiplier = plan->pc_shift = nullptr;
        return EH_OK;
    }
    EH_REQUIRE(count == plan->cout_caller, "per-channel: %d pairs for %d output channels", count, plan->cout_caller);
    int rc = check_perchannel(multipliers, shifts, count);
    if (rc) return rc;
    hipStream_t s = as_stream(stream);
    const size_t padded = (size_t)plan->cout + 4;  // the four-channel kernels read whole quads
    if (!plan->pc_multiplier && (rc = dev_alloc(&plan->pc_multiplier, padded))) return rc;
    if (!plan->pc_shift && (rc = dev_alloc(&plan->pc_shift, padded))) return rc;
    plan->pc_fast = all_pairs_fast(multipliers, shifts, count);
    return upload_padded_pairs(plan->pc_multiplier, plan->pc_shift, multipliers, shifts, count, 4, s);
}

int eh_dwconv2d_u8_repack(eh_dwconv_plan *plan, const void *weight, const void *bias, const eh_requant *q, void *stream) {
    EH_REQUIRE(plan != nullptr, "null plan");
    int rc = check_requant(q, plan->w_signed, plan->io_signed);
    if (rc) return rc;
    if ((rc = dw_set_weights(plan, weight, bias, as_stream(stream)))) return rc;
    return dw_refold(plan, *q, as_stream(stream));
}

// the kernel argument of a depthwise plan whose packed arrays match plan->q (after dw_refold)
static DwProblem dw_problem(const eh_dwconv_plan *plan, const void *input, void *output) {
    const eh_conv_desc &d = plan->d;
    DwProblem p;
    p.in = static_cast<const uint8_t *>(input);
    p.w = plan->w_copy;
    p.bias = plan->has_bias ? plan->bias_copy : nullptr;
    p.w_pair = plan->w_pair;
    p.bias_folded = plan->bias_folded;
    p.out = static_cast<uint8_t *>(output);
    p.n = d.n;
    p.c = d.c;
    p.h = d.h;
    p.w_ = d.w;
    p.cout = plan->cout;
    p.dm = d.depth_multiplier;
    p.kh = d.kh;
    p.kw = d.kw;
    p.stride_h = d.stride_h;
    p.stride_w = d.stride_w;
    p.pad_t = d.pad_t;
    p.pad_l = d.pad_l;
    p.dil_h = d.dil_h;
    p.dil_w = d.dil_w;
    p.ho = plan->ho;
    p.wo = plan->wo;
    p.zp_in = plan->q.zp_in;
    p.zp_w = plan->q.zp_w;
    p.w_signed = plan->w_signed ? 1 : 0;
    p.w_trip = plan->trip_valid ? plan->w_trip : nullptr;
    p.bias_trip = plan->bias_trip;
    p.w_fold = plan->fold_valid ? plan->w_fold : nullptr;
    p.bias_fold = plan->bias_fold;
    p.w_foldk = plan->foldk_valid ? plan->w_foldk : nullptr;
    p.bias_foldk = plan->bias_foldk;
    p.io_flip = plan->io_signed ? 0x80808080u : 0u;
    p.rq = make_requant_dev(plan->q);
    if (plan->pc_multiplier) {
        p.rq.pc_multiplier = plan->pc_multiplier;
        p.rq.pc_shift = plan->pc_shift;
        p.rq.fast = plan->pc_fast ? channel_fast_mode(plan->q) : 0;
    }
    return p;
}

int eh_dwconv2d_u8_run(eh_dwconv_plan *plan, const void *input, void *output, const eh_requant *q, void *stream) {
    EH_REQUIRE(plan != nullptr, "null plan");
    int rc = check_requant(q, plan->w_signed, plan->io_signed);
    if (rc) return rc;
    const eh_conv_desc &d = plan->d;
    if (d.n == 0) return EH_OK;
    EH_REQUIRE(input != nullptr && output != nullptr, "input/output pointer is null");
    hipStream_t s = as_stream(stream);
    if ((rc = dw_refold(plan, *q, s))) return rc;
    if (plan->rep_dm) {
        // (multiplier 1: only the rows' tails are new, and the copy reads whole dwords)
        rc = plan->rep_dm == 1 ? launch_pad_channels(static_cast<const uint8_t *>(input), plan->stage_in, (int64_t)d.n * d.h * d.w, 1, plan->rep_c, plan->cout, 0, s)
                               : launch_replicate_channels(static_cast<const uint8_t *>(input), plan->stage_in, (int64_t)d.n * d.h * d.w, plan->rep_c,
                                                           plan->rep_dm, plan->cout, s);
        if (rc) return rc;
        if (plan->cout != plan->cout_caller) {
            if ((rc = launch_dwconv_nhwc(dw_problem(plan, plan->stage_in, plan->stage_out), s))) return rc;
            return launch_keep_channels(plan->stage_out, static_cast<uint8_t *>(output), (int64_t)d.n * plan->ho * plan->wo, plan->cout,
                                        plan->cout_caller, s);
        }
        input = plan->stage_in;
    } else if (plan->planar) {
        if ((rc = launch_nchw2nhwc(static_cast<const uint8_t *>(input), plan->stage_in, d.n, d.c, d.h * d.w, s))) return rc;
        if ((rc = launch_dwconv_nhwc(dw_problem(plan, plan->stage_in, plan->stage_out), s))) return rc;
        return launch_nhwc2nchw(plan->stage_out, static_cast<uint8_t *>(output), d.n, plan->cout, plan->ho * plan->wo, s);
    }
    const DwProblem p = dw_problem(plan, input, output);
    return d.layout == EH_NHWC ? launch_dwconv_nhwc(p, s) : launch_dwconv_nchw(p, s);
}

int eh_dwconv2d_u8_destroy(eh_dwconv_plan *plan) {
    if (plan) {
        dw_release(plan);
        delete plan;
    }
    return EH_OK;
}


// ------------------------------------------------------------ pointwise + depthwise block

int eh_conv_dw_block_applies(const eh_conv_plan *pointwise, const eh_dwconv_plan *depthwise) {
    if (pointwise == nullptr || depthwise == nullptr) return 0;
    const GemmOp &op = pointwise->op;
    if (op.parts.size() != 1 || op.layout != EH_NHWC || op.io_signed) return 0;
    // (a plan that reads a channel-padded copy of its input, or shares its reduction between workgroups, runs as itself)
    if (op.pad_cg_to != 0 || op.parts[0].slices != 0) return 0;
    if (depthwise->d.layout != EH_NHWC || depthwise->io_signed || depthwise->rep_dm || depthwise->planar) return 0;
    if ((op.pc_multiplier != nullptr) != (depthwise->pc_multiplier != nullptr)) return 0;  // one pair per operator, or one per channel in both
    if (depthwise->d.n != pointwise->d.n || !(depthwise->w_trip || depthwise->w_fold)) return 0;
    // geometry and kernel family are checked on the problems themselves; the pointers and parameters of a run do not enter
    const GemmProblem pw = op.problem(op.parts[0], nullptr, nullptr, nullptr, nullptr);
    const DwProblem dw = dw_problem(depthwise, nullptr, nullptr);
    return pwdw_block_applies(pw, dw) ? 1 : 0;
}

int eh_conv_dw_block_listed(int32_t images, int32_t image_h, int32_t image_w, int32_t in_channels, int32_t expanded_channels, int32_t stride) {
    return pwdw_block_listed(images, image_h, image_w, in_channels, expanded_channels, stride) ? 1 : 0;
}

int eh_conv_dw_block_preferred(const eh_conv_plan *pointwise, const eh_dwconv_plan *depthwise) {
    if (!eh_conv_dw_block_applies(pointwise, depthwise)) return 0;
    const GemmOp &op = pointwise->op;
    const GemmProblem pw = op.problem(op.parts[0], nullptr, nullptr, nullptr, nullptr);
    const DwProblem dw = dw_problem(depthwise, nullptr, nullptr);
    return pwdw_block_preferred(pw, dw) ? 1 : 0;
}

int eh_conv_dw_block_run(eh_conv_plan *pointwise, eh_dwconv_plan *depthwise, const void *input, void *output,
                         const eh_requant *q_pointwise, const eh_requant *q_depthwise, int32_t rows_per_tile, int32_t cols_per_tile, void *stream) {
    EH_REQUIRE(pointwise != nullptr && depthwise != nullptr, "null plan");
    EH_REQUIRE(eh_conv_dw_block_applies(pointwise, depthwise), "block: these two plans do not fit the fused kernel");
    int rc = check_requant(q_pointwise, pointwise->op.w_signed, false);
    if (rc) return rc;
    if ((rc = check_requant(q_depthwise, depthwise->w_signed, false))) return rc;
    EH_REQUIRE(q_pointwise->zp_out == q_depthwise->zp_in, "block: the pointwise output zero point %d is not the depthwise input zero point %d",
               q_pointwise->zp_out, q_depthwise->zp_in);
    if (pointwise->d.n == 0) return EH_OK;
    EH_REQUIRE(input != nullptr && output != nullptr, "input/output pointer is null");
    hipStream_t s = as_stream(stream);
    if ((rc = pointwise->op.refold(*q_pointwise, s))) return rc;
    if ((rc = dw_refold(depthwise, *q_depthwise, s))) return rc;
    const GemmProblem pw = pointwise->op.problem(pointwise->op.parts[0], static_cast<const uint8_t *>(input), nullptr, nullptr, nullptr);
    const DwProblem dw = dw_problem(depthwise, nullptr, output);
    return launch_pwdw_block(pw, dw, rows_per_tile, cols_per_tile, s);
}

}  // extern "C"
