// Quantized residual Add and AveragePool on uint8 tensors (gfx950): the two
// operators a quantized MobileNet-style network needs between its convolutions.
// Both are plain HBM streaming kernels.
//
// Add follows the reference's quantized add (parameter derivation
// gpu/operators/cl_optimized_impls/CLAddQuantized.cpp:70-115, kernel
// gpu/operators/cl_kernels/AddKernelsQauntized.cpp:135-215): both inputs are
// shifted left by 20 bits, brought to a common scale by a Q31 multiplier and a
// rounding right shift each, summed, rescaled to the output the same way, offset
// and clamped.  AveragePool follows gpu/operators/cl_kernels/AveragepoolKernels.cpp:8-44:
// the window is clipped to the image, (sum + count / 2) / count, clamp.
#include "eh_internal.h"

namespace eh {
namespace {

// 16 bytes per thread where the three pointers allow it, bytes for the tail
__global__ __launch_bounds__(256) void add_u8_kernel(const uint8_t *__restrict__ a, const uint8_t *__restrict__ b,
                                                     uint8_t *__restrict__ out, const int64_t count, const int64_t vec_count,
                                                     const AddDev q) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < vec_count) {
        const uint4 va = reinterpret_cast<const uint4 *>(a)[i], vb = reinterpret_cast<const uint4 *>(b)[i];
        uint4 r;
        r.x = add_word(va.x, vb.x, q);
        r.y = add_word(va.y, vb.y, q);
        r.z = add_word(va.z, vb.z, q);
        r.w = add_word(va.w, vb.w, q);
        reinterpret_cast<uint4 *>(out)[i] = r;
    } else {
        const int64_t j = vec_count * 16 + (i - vec_count);
        if (j < count) out[j] = (uint8_t)add_one(a[j], b[j], q);
    }
}

struct PoolDev {
    int32_t n, c, h, w, ho, wo, kh, kw, stride_h, stride_w, pad_t, pad_l, act_min, act_max;
    uint32_t flip;  // 0x80808080 for int8 tensors: stored byte ^ 0x80 = value + 128
    FastDiv div_cq, div_wo, div_ho, div_full;  // by c / 4, wo, ho and kh * kw (launches of fewer than 2^31 threads)
};

// Window sum over (value + 128 for int8 tensors) to the stored output byte.  uint8: (sum + n/2) / n.  int8: the sum of
// the signed values, rounded half away from zero (SIGNEDavepooling_tflite,
// gpu/operators/cl_kernels/AveragepoolKernels.cpp:70-74), which differs from the uint8 rule at negative ties.
__device__ __forceinline__ uint32_t pool_finish(int s, int cnt, const PoolDev &p) {
    int v = 0;
    if (cnt > 0) {
        if (p.flip) {
            s -= 128 * cnt;
            v = s > 0 ? (s + cnt / 2) / cnt : (s - cnt / 2) / cnt;
        } else {
            v = (s + cnt / 2) / cnt;
        }
    }
    v = v < p.act_min ? p.act_min : v;
    v = v > p.act_max ? p.act_max : v;
    return (uint32_t)v & 255u;
}

// channels-last: ROWS threads (adjacent lanes) own four consecutive channels of one output pixel (c % 4 == 0) and
// share the window's rows; ROWS = 8 serves launches with few outputs and tall windows (a global pool is one long
// chain of dependent loads otherwise), ROWS = 1 the rest
template <int ROWS>
__global__ __launch_bounds__(256) void avgpool_nhwc_vec4_kernel(const uint8_t *__restrict__ in, uint8_t *__restrict__ out,
                                                                const PoolDev p, const int64_t total) {
    const int64_t tid = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t idx = tid / ROWS;
    const int part = (int)(tid % ROWS);
    const bool live = idx < total;  // whole groups of ROWS lanes are live or not; all lanes reach the shuffles
    const int cq = p.c >> 2;
    const int c4 = live ? (int)(idx % cq) : 0;
    int64_t r = live ? idx / cq : 0;
    const int ox = (int)(r % p.wo);
    r /= p.wo;
    const int oy = (int)(r % p.ho), img = (int)(r / p.ho);
    int y0 = oy * p.stride_h - p.pad_t, x0 = ox * p.stride_w - p.pad_l;
    const int y1 = y0 + p.kh < p.h ? y0 + p.kh : p.h, x1 = x0 + p.kw < p.w ? x0 + p.kw : p.w;
    y0 = y0 < 0 ? 0 : y0;
    x0 = x0 < 0 ? 0 : x0;
    const int cnt = (y1 - y0) * (x1 - x0);
    int s0 = 0, s1 = 0, s2 = 0, s3 = 0;
    auto take = [&](uint32_t v) {
        v ^= p.flip;
        s0 += v & 255u;
        s1 += (v >> 8) & 255u;
        s2 += (v >> 16) & 255u;
        s3 += v >> 24;
    };
    // eight window pixels are requested before the first is summed
    for (int y = y0 + part; y < y1 && live; y += ROWS) {
        const uint8_t *row = in + ((size_t)img * p.h + y) * p.w * p.c + c4 * 4;
        int x = x0;
        for (; x + 8 <= x1; x += 8) {
            uint32_t v[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) v[t] = *reinterpret_cast<const uint32_t *>(row + (size_t)(x + t) * p.c);
#pragma unroll
            for (int t = 0; t < 8; ++t) take(v[t]);
        }
        uint32_t v[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) v[t] = x + t < x1 ? *reinterpret_cast<const uint32_t *>(row + (size_t)(x + t) * p.c) : p.flip;
#pragma unroll
        for (int t = 0; t < 8; ++t) take(v[t]);
    }
#pragma unroll
    for (int step = 1; step < ROWS; step <<= 1) {
        s0 += __shfl_xor(s0, step);
        s1 += __shfl_xor(s1, step);
        s2 += __shfl_xor(s2, step);
        s3 += __shfl_xor(s3, step);
    }
    if (live && part == 0)
        *reinterpret_cast<uint32_t *>(out + idx * 4) = pool_finish(s0, cnt, p) | (pool_finish(s1, cnt, p) << 8) |
                                                       (pool_finish(s2, cnt, p) << 16) | (pool_finish(s3, cnt, p) << 24);
}

// The same for launches of fewer than 2^31 threads, which is all but absurd ones: 32-bit indices decoded with
// multiplications (the 64-bit divisions of the kernel above cost more than a small window's loads and sums together:
// a 2x2 stride-2 pool of 64 x 112 x 112 x 64 took 34 us for 64 MB), the division by the window size as a multiplication
// wherever the window lies wholly inside the image, and a window row fetched four pixels at a time.
template <int ROWS>
__global__ __launch_bounds__(256) void avgpool_nhwc_vec4_small_index_kernel(const uint8_t *__restrict__ in, uint8_t *__restrict__ out,
                                                                            const PoolDev p, const uint32_t total) {
    const uint32_t tid = blockIdx.x * 256u + threadIdx.x;
    const uint32_t idx = tid / ROWS;
    const int part = (int)(tid % ROWS);
    const bool live = idx < total;  // whole groups of ROWS lanes are live or not; all lanes reach the shuffles
    const uint32_t cq = (uint32_t)p.c >> 2;
    uint32_t r = live ? fastdiv(idx, p.div_cq) : 0u;
    const uint32_t c4 = live ? idx - r * cq : 0u;
    const uint32_t r1 = fastdiv(r, p.div_wo);
    const int ox = (int)(r - r1 * (uint32_t)p.wo);
    const uint32_t img = fastdiv(r1, p.div_ho);
    const int oy = (int)(r1 - img * (uint32_t)p.ho);
    int y0 = oy * p.stride_h - p.pad_t, x0 = ox * p.stride_w - p.pad_l;
    const int y1 = y0 + p.kh < p.h ? y0 + p.kh : p.h, x1 = x0 + p.kw < p.w ? x0 + p.kw : p.w;
    y0 = y0 < 0 ? 0 : y0;
    x0 = x0 < 0 ? 0 : x0;
    const int cnt = (y1 - y0) * (x1 - x0);
    int s0 = 0, s1 = 0, s2 = 0, s3 = 0;
    auto take = [&](uint32_t v) {
        v ^= p.flip;
        s0 += v & 255u;
        s1 += (v >> 8) & 255u;
        s2 += (v >> 16) & 255u;
        s3 += v >> 24;
    };
    const size_t row_bytes = (size_t)p.w * p.c;
    for (int y = y0 + part; y < y1 && live; y += ROWS) {
        const uint8_t *row = in + ((size_t)img * p.h + y) * row_bytes + c4 * 4;
        for (int x = x0; x < x1; x += 4) {  // four window pixels are requested before the first is summed
            uint32_t v[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) v[t] = x + t < x1 ? *reinterpret_cast<const uint32_t *>(row + (size_t)(x + t) * p.c) : p.flip;
#pragma unroll
            for (int t = 0; t < 4; ++t) take(v[t]);
        }
    }
#pragma unroll
    for (int step = 1; step < ROWS; step <<= 1) {
        s0 += __shfl_xor(s0, step);
        s1 += __shfl_xor(s1, step);
        s2 += __shfl_xor(s2, step);
        s3 += __shfl_xor(s3, step);
    }
    if (live && part == 0) {
        uint32_t o;
        if (cnt == p.kh * p.kw && !p.flip) {  // the whole window, uint8 rule: (sum + n / 2) / n with the division as a multiplication
            const uint32_t half = (uint32_t)cnt >> 1;
            auto fin = [&](int sum) {
                int v = (int)fastdiv((uint32_t)sum + half, p.div_full);
                v = v < p.act_min ? p.act_min : v;
                v = v > p.act_max ? p.act_max : v;
                return (uint32_t)v & 255u;
            };
            o = fin(s0) | (fin(s1) << 8) | (fin(s2) << 16) | (fin(s3) << 24);
        } else {
            o = pool_finish(s0, cnt, p) | (pool_finish(s1, cnt, p) << 8) | (pool_finish(s2, cnt, p) << 16) | (pool_finish(s3, cnt, p) << 24);
        }
        *reinterpret_cast<uint32_t *>(out + (size_t)idx * 4) = o;
    }
}

// one output element per thread, either layout
template <bool NHWC>
__global__ __launch_bounds__(256) void avgpool_scalar_kernel(const uint8_t *__restrict__ in, uint8_t *__restrict__ out,
                                                             const PoolDev p, const int64_t total) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    int ch, ox, oy, img;
    int64_t r = idx;
    if (NHWC) {
        ch = (int)(r % p.c);
        r /= p.c;
        ox = (int)(r % p.wo);
        r /= p.wo;
        oy = (int)(r % p.ho);
        img = (int)(r / p.ho);
    } else {
        ox = (int)(r % p.wo);
        r /= p.wo;
        oy = (int)(r % p.ho);
        r /= p.ho;
        ch = (int)(r % p.c);
        img = (int)(r / p.c);
    }
    int y0 = oy * p.stride_h - p.pad_t, x0 = ox * p.stride_w - p.pad_l;
    const int y1 = y0 + p.kh < p.h ? y0 + p.kh : p.h, x1 = x0 + p.kw < p.w ? x0 + p.kw : p.w;
    y0 = y0 < 0 ? 0 : y0;
    x0 = x0 < 0 ? 0 : x0;
    const int cnt = (y1 - y0) * (x1 - x0);
    int s = 0;
    for (int y = y0; y < y1; ++y)
        for (int x = x0; x < x1; ++x)
            s += (NHWC ? in[(((size_t)img * p.h + y) * p.w + x) * p.c + ch] : in[(((size_t)img * p.c + ch) * p.h + y) * p.w + x]) ^
                 (p.flip & 255u);
    out[idx] = (uint8_t)pool_finish(s, cnt, p);
}

}  // namespace

int check_add_requant(const eh_add_requant *q) {
    EH_REQUIRE(q != nullptr, "add: null parameters");
    EH_REQUIRE(q->mult_a >= 0 && q->mult_b >= 0 && q->mult_out >= 0, "add: negative multiplier");
    EH_REQUIRE(q->left_shift >= 0 && q->left_shift <= 23, "add: left shift %d outside [0, 23]", q->left_shift);
    EH_REQUIRE(q->shift_a >= -31 && q->shift_b >= -31 && q->shift_out >= -31, "add: shift below -31");
    EH_REQUIRE(q->act_min >= 0 && q->act_max <= 255 && q->act_min <= q->act_max, "add: activation range [%d, %d] invalid",
               q->act_min, q->act_max);
    return EH_OK;
}

int launch_add_u8(const uint8_t *a, const uint8_t *b, uint8_t *out, int64_t count, const AddDev &d, hipStream_t stream) {
    if (count <= 0) return EH_OK;
    const bool wide = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    const int64_t vec_count = wide ? count / 16 : 0;
    const int64_t threads = vec_count + (count - vec_count * 16);
    const int64_t blocks = (threads + 255) / 256;
    EH_REQUIRE(blocks < (1ll << 31), "add: tensor too large");
    hipLaunchKernelGGL(add_u8_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, a, b, out, count, vec_count, d);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

}  // namespace eh

using namespace eh;

extern "C" {

void eh_make_add_requant(float scale_a, int32_t zp_a, float scale_b, int32_t zp_b, float scale_out, int32_t zp_out,
                         int activation, int activation_enabled, eh_add_requant *out) {
    out->zp_a = zp_a;
    out->zp_b = zp_b;
    out->zp_out = zp_out;
    out->left_shift = 20;
    const float mx = scale_a > scale_b ? scale_a : scale_b;  // the maximum is taken in float, then widened
    const double twice_max = 2 * (double)mx;
    eh_quantize_multiplier((double)scale_a / twice_max, &out->mult_a, &out->shift_a);
    eh_quantize_multiplier((double)scale_b / twice_max, &out->mult_b, &out->shift_b);
    eh_quantize_multiplier(twice_max / ((double)(1 << out->left_shift) * (double)scale_out), &out->mult_out, &out->shift_out);
    out->act_min = 0;
    out->act_max = 255;
    if (activation_enabled) eh_act_range_u8(activation, scale_out, zp_out, &out->act_min, &out->act_max);
}

int eh_add_u8(const void *a, const void *b, void *out, int64_t count, const eh_add_requant *q, void *stream) {
    EH_REQUIRE(q != nullptr, "add: null parameters");
    EH_REQUIRE(count >= 0, "add: negative count");
    if (count == 0) return EH_OK;
    EH_REQUIRE(a && b && out, "add: null tensor");
    int rc = check_add_requant(q);
    if (rc) return rc;
    return launch_add_u8(static_cast<const uint8_t *>(a), static_cast<const uint8_t *>(b), static_cast<uint8_t *>(out), count,
                         make_add_dev(*q), reinterpret_cast<hipStream_t>(stream));
}

int eh_avgpool_u8(const void *in, void *out, const eh_pool_desc *desc, void *stream) {
    EH_REQUIRE(desc != nullptr, "avgpool: null descriptor");
    eh_pool_desc d = *desc;
    const bool io_signed = (d.layout & EH_IO_SIGNED) != 0;
    d.layout &= ~EH_IO_SIGNED;
    EH_REQUIRE(d.n >= 0 && d.c >= 0 && d.h >= 0 && d.w >= 0, "avgpool: negative extent");
    EH_REQUIRE(d.kh > 0 && d.kw > 0 && d.stride_h > 0 && d.stride_w > 0, "avgpool: bad window or stride");
    EH_REQUIRE(d.pad_t >= 0 && d.pad_b >= 0 && d.pad_l >= 0 && d.pad_r >= 0, "avgpool: negative padding");
    EH_REQUIRE(d.layout == EH_NCHW || d.layout == EH_NHWC, "avgpool: bad layout %d", d.layout);
    EH_REQUIRE(d.act_min >= (io_signed ? -128 : 0) && d.act_max <= (io_signed ? 127 : 255) && d.act_min <= d.act_max,
               "avgpool: activation range [%d, %d] invalid", d.act_min, d.act_max);
    if ((int64_t)d.n * d.c * d.h * d.w == 0) return EH_OK;
    PoolDev p;
    p.n = d.n;
    p.c = d.c;
    p.h = d.h;
    p.w = d.w;
    p.ho = (d.h + d.pad_t + d.pad_b - d.kh) / d.stride_h + 1;
    p.wo = (d.w + d.pad_l + d.pad_r - d.kw) / d.stride_w + 1;
    EH_REQUIRE(d.h + d.pad_t + d.pad_b >= d.kh && d.w + d.pad_l + d.pad_r >= d.kw, "avgpool: window larger than the padded image");
    p.kh = d.kh;
    p.kw = d.kw;
    p.stride_h = d.stride_h;
    p.stride_w = d.stride_w;
    p.pad_t = d.pad_t;
    p.pad_l = d.pad_l;
    p.act_min = d.act_min;
    p.act_max = d.act_max;
    p.flip = io_signed ? 0x80808080u : 0u;
    EH_REQUIRE(in && out, "avgpool: null tensor");
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const int64_t outputs = (int64_t)d.n * d.c * p.ho * p.wo;
    const bool vec4 = d.layout == EH_NHWC && (d.c & 3) == 0 &&
                      ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 3) == 0;
    const int64_t total = vec4 ? outputs / 4 : outputs;
    const bool split_rows = vec4 && total < 256 * 1024 && d.kh >= 4;  // few threads, tall windows: eight lanes per output
    const int64_t blocks = ((split_rows ? total * 8 : total) + 255) / 256;
    EH_REQUIRE(blocks < (1ll << 31), "avgpool: tensor too large");
    if (vec4 && blocks * 256 < (1ll << 31) && p.ho > 0 && p.wo > 0 && total > 0) {
        p.div_cq = make_fastdiv((uint32_t)(d.c >> 2));
        p.div_wo = make_fastdiv((uint32_t)p.wo);
        p.div_ho = make_fastdiv((uint32_t)p.ho);
        p.div_full = make_fastdiv((uint32_t)(d.kh * d.kw));
        if (split_rows)
            hipLaunchKernelGGL(avgpool_nhwc_vec4_small_index_kernel<8>, dim3((unsigned)blocks), dim3(256), 0, s, static_cast<const uint8_t *>(in),
                               static_cast<uint8_t *>(out), p, (uint32_t)total);
        else
            hipLaunchKernelGGL(avgpool_nhwc_vec4_small_index_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, s, static_cast<const uint8_t *>(in),
                               static_cast<uint8_t *>(out), p, (uint32_t)total);
        EH_HIP(hipGetLastError());
        return EH_OK;
    }
    if (split_rows)
        hipLaunchKernelGGL(avgpool_nhwc_vec4_kernel<8>, dim3((unsigned)blocks), dim3(256), 0, s, static_cast<const uint8_t *>(in),
                           static_cast<uint8_t *>(out), p, total);
    else if (vec4)
        hipLaunchKernelGGL(avgpool_nhwc_vec4_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, s, static_cast<const uint8_t *>(in),
                           static_cast<uint8_t *>(out), p, total);
    else if (d.layout == EH_NHWC)
        hipLaunchKernelGGL(avgpool_scalar_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, s,
                           static_cast<const uint8_t *>(in), static_cast<uint8_t *>(out), p, total);
    else
        hipLaunchKernelGGL(avgpool_scalar_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, s,
                           static_cast<const uint8_t *>(in), static_cast<uint8_t *>(out), p, total);
    EH_HIP(hipGetLastError());
    return EH_OK;
}

}  // extern "C"
