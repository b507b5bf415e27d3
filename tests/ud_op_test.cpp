// Operator-level tests of the HIP userdriver backend, shaped like the reference's
// op tests (src/userdriver/gpu/op_test/convolution_test.cpp:16-267,
// fullyconnected_test.cpp:12-120): build tensors from host arrays, initialize /
// execute / release an operator, read the output back and compare it, here bit for
// bit against the CPU oracle.  The oracle (oracle/eden_oracle.h) is linked into
// this test program only; the operator classes never see it.
//
//   ud_op_test              run everything (needs the GPU)
//   ud_op_test --host-only  buffer-pool bookkeeping and argument checks that touch no device
//   ud_op_test --filter T   only the tests whose name contains T
#include <cstdio>
#include <cstring>
#include <functional>
#include <string>
#include <vector>

#include "HipOpConstructor.hpp"
#include "HipOperators.hpp"
#include "HipUserDriver.hpp"
#include "eden_oracle.h"
#include "userdriver_operator.hpp"

using namespace enn::ud;
using namespace enn::ud::hip;

static int g_failed = 0, g_run = 0;
static const char *g_filter = nullptr;  // --filter TEXT: run only the tests whose name contains TEXT
#define EXPECT(cond)                                                                    \
    do {                                                                                \
        if (!(cond)) {                                                                  \
            std::printf("    EXPECT failed at line %d: %s\n", __LINE__, #cond);        \
            ok = false;                                                                 \
        }                                                                               \
    } while (0)

static void run_test(const char *name, const std::function<bool()> &fn) {
    if (g_filter && !std::strstr(name, g_filter)) return;
    std::printf("[ RUN  ] %s\n", name);
    std::fflush(stdout);
    ++g_run;
    const bool ok = fn();
    if (!ok) ++g_failed;
    std::printf("[ %s ] %s\n", ok ? " OK " : "FAIL", name);
    std::fflush(stdout);
}

static std::vector<uint8_t> rand_u8(size_t n, uint64_t seed, int lo = 0, int hi = 255) {
    std::vector<uint8_t> v(n);
    eo_fill_u8(v.data(), (int64_t)n, seed, lo, hi);
    return v;
}
static std::vector<int32_t> rand_i32(size_t n, uint64_t seed, int lo, int hi) {
    std::vector<int32_t> v(n);
    eo_fill_i32(v.data(), (int64_t)n, seed, lo, hi);
    return v;
}
static bool same(const std::vector<uint8_t> &a, const std::vector<uint8_t> &b) {
    if (a.size() != b.size()) return false;
    size_t bad = 0, first = 0;
    for (size_t i = 0; i < a.size(); ++i)
        if (a[i] != b[i] && bad++ == 0) first = i;
    if (bad) {
        std::printf("    %zu of %zu bytes differ; first at %zu: got %u want %u\n", bad, a.size(), first, a[first], b[first]);
        std::printf("    got :");
        for (size_t i = first; i < a.size() && i < first + 16; ++i) std::printf(" %3u", a[i]);
        std::printf("\n    want:");
        for (size_t i = first; i < b.size() && i < first + 16; ++i) std::printf(" %3u", b[i]);
        std::printf("\n");
    }
    return bad == 0;
}
static bool varied(const std::vector<uint8_t> &v) {
    int seen[256] = {0}, distinct = 0;
    for (uint8_t x : v)
        if (!seen[x]++) ++distinct;
    return distinct > 8;
}
static std::vector<uint8_t> nchw_to_nhwc(const std::vector<uint8_t> &x, int n, int c, int h, int w) {
    std::vector<uint8_t> y(x.size());
    eo_nchw2nhwc_u8(x.data(), y.data(), n, c, h, w);
    return y;
}
static std::vector<uint8_t> nhwc_to_nchw(const std::vector<uint8_t> &x, int n, int c, int h, int w) {
    std::vector<uint8_t> y(x.size());
    eo_nhwc2nchw_u8(x.data(), y.data(), n, c, h, w);
    return y;
}
static eo_conv_shape shape(int n, int c, int h, int w, int cout, int kh, int kw, int sh = 1, int sw = 1, int pt = 0, int pb = 0,
                           int pl = 0, int pr = 0, int dh = 1, int dw = 1, int groups = 1, int dm = 1) {
    eo_conv_shape s = {n, c, h, w, cout, kh, kw, sh, sw, pt, pb, pl, pr, dh, dw, groups, dm};
    return s;
}

static const PrecisionType U8 = PrecisionType::UINT8;
struct Quant {
    float s_in, s_w, s_out;
    int zp_in, zp_w, zp_out;
    float s_bias() const { return s_in * s_w; }  // float32 product, as a converter would store it
};

// ---------------------------------------------------------------- convolution

static bool conv_case(const std::shared_ptr<HipRuntime> &rt, const eo_conv_shape &s, const Quant &qt, ActivationInfo act,
                      bool nchw, bool androidNN, uint64_t seed) {
    bool ok = true;
    const int ho = eo_conv_out_dim(s.h, s.pad_t, s.pad_b, s.kh, s.dil_h, s.stride_h);
    const int wo = eo_conv_out_dim(s.w, s.pad_l, s.pad_r, s.kw, s.dil_w, s.stride_w);
    const int cig = s.c / s.groups;
    auto x = rand_u8((size_t)s.n * s.c * s.h * s.w, seed);
    auto w = rand_u8((size_t)s.cout * cig * s.kh * s.kw, seed + 1);
    auto b = rand_i32(s.cout, seed + 2, -1000, 1000);
    eo_quant q;
    eo_make_quant(qt.s_in, qt.zp_in, qt.s_w, qt.zp_w, qt.s_bias(), qt.s_out, qt.zp_out, (int)act.activation(), act.isEnabled(), &q);
    std::vector<uint8_t> want((size_t)s.n * s.cout * ho * wo);
    eo_conv2d_u8(x.data(), w.data(), b.data(), want.data(), &s, &q, nullptr);

    // tensors as the model hands them over: planar, or channels-last with positional dims
    const bool ohwi = androidNN || !nchw;
    Dim4 in_dim = nchw ? Dim4{(uint32_t)s.n, (uint32_t)s.c, (uint32_t)s.h, (uint32_t)s.w}
                       : Dim4{(uint32_t)s.n, (uint32_t)s.h, (uint32_t)s.w, (uint32_t)s.c};
    Dim4 out_dim = nchw ? Dim4{(uint32_t)s.n, (uint32_t)s.cout, (uint32_t)ho, (uint32_t)wo}
                        : Dim4{(uint32_t)s.n, (uint32_t)ho, (uint32_t)wo, (uint32_t)s.cout};
    Dim4 w_dim = ohwi ? Dim4{(uint32_t)s.cout, (uint32_t)s.kh, (uint32_t)s.kw, (uint32_t)cig}
                      : Dim4{(uint32_t)s.cout, (uint32_t)cig, (uint32_t)s.kh, (uint32_t)s.kw};
    std::vector<uint8_t> w_dev = ohwi ? nchw_to_nhwc(w, s.cout, cig, s.kh, s.kw) : w;
    const DataOrder order = nchw ? DataOrder::NCHW : DataOrder::NHWC;
    std::shared_ptr<ITensor> input = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, in_dim, order, qt.s_in, qt.zp_in);
    std::shared_ptr<ITensor> weight = std::make_shared<HipTensor>(rt, U8, w_dev.data(), w_dim, order, qt.s_w, qt.zp_w);
    std::shared_ptr<ITensor> bias = std::make_shared<HipTensor>(rt, U8, b.data(), Dim4{1, (uint32_t)s.cout, 1, 1}, DataOrder::NCHW, qt.s_bias(), 0);
    std::shared_ptr<ITensor> output = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, out_dim, order, qt.s_out, qt.zp_out);

    auto params = std::make_shared<ConvolutionParameters>();
    params->padding = {(uint32_t)s.pad_t, (uint32_t)s.pad_r, (uint32_t)s.pad_b, (uint32_t)s.pad_l};
    params->dilation = {(uint32_t)s.dil_h, (uint32_t)s.dil_w};
    params->stride = {(uint32_t)s.stride_h, (uint32_t)s.stride_w};
    params->group_size = s.groups;
    params->androidNN = androidNN;
    params->isNCHW = nchw;
    params->activation_info = std::make_shared<ActivationInfo>(act);

    HipConvolution conv(rt, U8);
    EXPECT(conv.initialize({input, weight, bias}, {output}, params) == Status::SUCCESS);
    rt->assignBufferPool();
    std::vector<uint8_t> x_dev = nchw ? x : nchw_to_nhwc(x, s.n, s.c, s.h, s.w);
    EXPECT(input->writeData(x_dev.data()) == Status::SUCCESS);
    EXPECT(conv.execute() == Status::SUCCESS);
    std::vector<uint8_t> got(want.size());
    EXPECT(output->readData(got.data()) == Status::SUCCESS);
    if (!nchw) got = nhwc_to_nchw(got, s.n, s.cout, ho, wo);
    EXPECT(same(got, want));
    EXPECT(varied(want));
    EXPECT(conv.release() == Status::SUCCESS);
    return ok;
}

// ---------------------------------------------------------------- tests

// One execution of a built list the way the userdriver does it: host bytes into the list's inputs, the executor,
// the outputs back (gpu_userdriver.cc:97-103).
static EnnReturn run_list(OperationConstructor &built, OperationExecutor &executor, const std::vector<const void *> &inputs,
                          const std::vector<void *> &outputs) {
    if (inputs.size() != built.in_tensors.size() || outputs.size() != built.out_tensors.size()) return ENN_RET_FAILED;
    for (size_t i = 0; i < inputs.size(); ++i)
        if (built.in_tensors[i]->writeData(const_cast<void *>(inputs[i]), false) != Status::SUCCESS) return ENN_RET_FAILED;
    UDBuffers buffers;
    BufferTable table;
    if (executor.execute(built.operators, buffers, table) != ENN_RET_SUCCESS) return ENN_RET_FAILED;
    for (size_t i = 0; i < outputs.size(); ++i)
        if (built.out_tensors[i]->readData(outputs[i], true) != Status::SUCCESS) return ENN_RET_FAILED;
    return ENN_RET_SUCCESS;
}

static int gpu_tests() {
    auto lib = std::make_shared<HipComputeLibrary>(0);
    if (!lib->valid() || lib->initialize_queue() != Status::SUCCESS) {
        std::printf("cannot initialise the GPU runtime: %s\n", eh_last_error());
        return 2;
    }
    auto rt = lib->runtime();
    const Quant q1 = {0.02f, 0.005f, 0.05f, 128, 120, 0};

    run_test("Convolution.Config1_3x3_64to64_56x56_nchw_relu", [&] {
        return conv_case(rt, shape(1, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1, 1, 1), q1, ActivationInfo(ActivationInfo::ActivationType::RELU, true), true, false, 0xEDF2);
    });
    run_test("Convolution.ChannelsLast_androidNN_weights_stride2", [&] {
        return conv_case(rt, shape(2, 32, 15, 17, 48, 3, 3, 2, 2, 0, 1, 0, 1), {0.02f, 0.005f, 0.04f, 100, 131, 7}, ActivationInfo(ActivationInfo::ActivationType::RELU6, true), false, true, 11);
    });
    run_test("Convolution.Planar_androidNN_weights", [&] {
        return conv_case(rt, shape(1, 16, 9, 9, 24, 3, 3, 1, 1, 1, 1, 1, 1), {0.02f, 0.005f, 0.02f, 100, 131, 7}, ActivationInfo(), true, true, 12);
    });
    run_test("Convolution.Grouped_dilated_3_channel_groups", [&] {
        return conv_case(rt, shape(1, 12, 10, 10, 12, 3, 3, 1, 1, 2, 2, 2, 2, 2, 2, 3), {0.02f, 0.005f, 0.08f, 120, 131, 128}, ActivationInfo(), true, false, 13);
    });
    run_test("Convolution.Pointwise_24_to_144_channels_last", [&] {
        return conv_case(rt, shape(2, 24, 28, 28, 144, 1, 1), {0.02f, 0.004f, 0.03f, 77, 140, 3}, ActivationInfo(ActivationInfo::ActivationType::RELU6, true), false, false, 14);
    });

    run_test("Convolution.BiasScaleMismatch_gives_clamped_zero_point", [&] {
        bool ok = true;
        auto x = rand_u8(1 * 16 * 6 * 6, 21), w = rand_u8(16 * 16 * 9, 22);
        auto b = rand_i32(16, 23, -1000, 1000);
        std::shared_ptr<ITensor> input = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{1, 16, 6, 6}, DataOrder::NCHW, 0.02f, 128);
        std::shared_ptr<ITensor> weight = std::make_shared<HipTensor>(rt, U8, w.data(), Dim4{16, 16, 3, 3}, DataOrder::NCHW, 0.005f, 120);
        // an int32 bias built without quantization parameters keeps scale 1.0 (gpu_op_constructor.cc:2032-2039)
        std::shared_ptr<ITensor> bias = std::make_shared<HipTensor>(rt, U8, b.data(), Dim4{1, 16, 1, 1});
        std::shared_ptr<ITensor> output = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{1, 16, 6, 6}, DataOrder::NCHW, 0.05f, 42);
        auto params = std::make_shared<ConvolutionParameters>();
        params->padding = {1, 1, 1, 1};
        HipConvolution conv(rt, U8);
        EXPECT(conv.initialize({input, weight, bias}, {output}, params) == Status::SUCCESS);
        EXPECT(input->writeData(x.data()) == Status::SUCCESS);
        EXPECT(conv.execute() == Status::SUCCESS);
        std::vector<uint8_t> got(16 * 36);
        EXPECT(output->readData(got.data()) == Status::SUCCESS);
        for (uint8_t v : got) EXPECT(v == 42);
        return ok;
    });

    run_test("Convolution.QuantParamsAreReadAtExecute_and_WeightsAsInput", [&] {
        bool ok = true;
        const eo_conv_shape s = shape(1, 16, 8, 8, 16, 3, 3, 1, 1, 1, 1, 1, 1);
        auto x = rand_u8(16 * 64, 31), w = rand_u8(16 * 16 * 9, 32), w2 = rand_u8(16 * 16 * 9, 33);
        auto b = rand_i32(16, 34, -1000, 1000);
        std::shared_ptr<ITensor> input = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{1, 16, 8, 8}, DataOrder::NCHW, 0.02f, 128);
        // weights as a run-time input: a shape-only tensor that is written afterwards
        std::shared_ptr<ITensor> weight = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{16, 16, 3, 3}, DataOrder::NCHW, 0.005f, 120);
        std::shared_ptr<ITensor> bias = std::make_shared<HipTensor>(rt, U8, b.data(), Dim4{1, 16, 1, 1}, DataOrder::NCHW, 0.02f * 0.005f, 0);
        std::shared_ptr<ITensor> output = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{1, 16, 8, 8}, DataOrder::NCHW, 0.05f, 10);
        EXPECT(!weight->is_const() && bias->is_const());
        auto params = std::make_shared<ConvolutionParameters>();
        params->padding = {1, 1, 1, 1};
        HipConvolution conv(rt, U8);
        EXPECT(weight->writeData(w.data()) == Status::SUCCESS);
        EXPECT(conv.initialize({input, weight, bias}, {output}, params) == Status::SUCCESS);
        EXPECT(input->writeData(x.data()) == Status::SUCCESS);
        std::vector<uint8_t> got(16 * 64), want(16 * 64);
        eo_quant q;
        auto check = [&](const std::vector<uint8_t> &wt, float s_out, int zp_in, int zp_out) {
            eo_make_quant(0.02f, zp_in, 0.005f, 120, 0.02f * 0.005f, s_out, zp_out, 0, 0, &q);
            eo_conv2d_u8(x.data(), wt.data(), b.data(), want.data(), &s, &q, nullptr);
            EXPECT(conv.execute() == Status::SUCCESS);
            EXPECT(output->readData(got.data()) == Status::SUCCESS);
            EXPECT(same(got, want));
        };
        check(w, 0.05f, 128, 10);
        input->setZeroPoint(99);   // the tensors are re-quantized between runs
        output->setScale(0.07f);
        output->setZeroPoint(20);
        check(w, 0.07f, 99, 20);
        EXPECT(weight->writeData(w2.data()) == Status::SUCCESS);  // new weights arrive as data
        check(w2, 0.07f, 99, 20);
        return ok;
    });

    run_test("DepthwiseConvolution.Config3_geometry_channels_last_and_planar", [&] {
        bool ok = true;
        for (int nchw = 0; nchw < 2; ++nchw) {
            const eo_conv_shape s = shape(2, 144, 56, 56, 144, 3, 3, 2, 2, 1, 1, 1, 1, 1, 1, 1, 1);
            const int ho = 28, wo = 28;
            auto x = rand_u8((size_t)2 * 144 * 56 * 56, 41), w = rand_u8(144 * 9, 42);
            auto b = rand_i32(144, 43, -1000, 1000);
            eo_quant q;
            eo_make_quant(0.03f, 17, 0.006f, 140, 0.03f * 0.006f, 0.025f, 9, EO_ACT_RELU6, 1, &q);
            std::vector<uint8_t> want((size_t)2 * 144 * ho * wo), got(want.size());
            eo_dwconv2d_u8(x.data(), w.data(), b.data(), want.data(), &s, &q, nullptr);
            const DataOrder order = nchw ? DataOrder::NCHW : DataOrder::NHWC;
            const Dim4 in_dim = nchw ? Dim4{2, 144, 56, 56} : Dim4{2, 56, 56, 144};
            const Dim4 out_dim = nchw ? Dim4{2, 144, 28, 28} : Dim4{2, 28, 28, 144};
            std::shared_ptr<ITensor> input = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, in_dim, order, 0.03f, 17);
            std::shared_ptr<ITensor> weight = std::make_shared<HipTensor>(rt, U8, w.data(), Dim4{144, 1, 3, 3}, DataOrder::NCHW, 0.006f, 140);
            std::shared_ptr<ITensor> bias = std::make_shared<HipTensor>(rt, U8, b.data(), Dim4{1, 144, 1, 1}, DataOrder::NCHW, 0.03f * 0.006f, 0);
            std::shared_ptr<ITensor> output = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, out_dim, order, 0.025f, 9);
            auto params = std::make_shared<DepthwiseConvolutionParameters>();
            params->padding = {1, 1, 1, 1};
            params->stride = {2, 2};
            params->isNCHW = nchw != 0;
            params->activation_info = std::make_shared<ActivationInfo>(ActivationInfo::ActivationType::RELU6, true);
            HipDepthwiseConvolution dw(rt, U8);
            EXPECT(dw.initialize({input, weight, bias}, {output}, params) == Status::SUCCESS);
            auto x_dev = nchw ? x : nchw_to_nhwc(x, 2, 144, 56, 56);
            EXPECT(input->writeData(x_dev.data()) == Status::SUCCESS);
            EXPECT(dw.execute() == Status::SUCCESS);
            EXPECT(output->readData(got.data()) == Status::SUCCESS);
            if (!nchw) got = nhwc_to_nchw(got, 2, 144, ho, wo);
            EXPECT(same(got, want));
            EXPECT(varied(want));
            EXPECT(dw.release() == Status::SUCCESS);
        }
        return ok;
    });

    run_test("DepthwiseConvolution.DepthMultiplier2", [&] {
        bool ok = true;
        const eo_conv_shape s = shape(1, 8, 9, 7, 16, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, 2);
        auto x = rand_u8(8 * 63, 51), w = rand_u8(16 * 9, 52);
        auto b = rand_i32(16, 53, -100, 100);
        eo_quant q;
        eo_make_quant(0.03f, 17, 0.006f, 140, 0.03f * 0.006f, 0.02f, 128, 0, 0, &q);
        std::vector<uint8_t> want(16 * 63), got(16 * 63);
        eo_dwconv2d_u8(x.data(), w.data(), b.data(), want.data(), &s, &q, nullptr);
        std::shared_ptr<ITensor> input = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{1, 8, 9, 7}, DataOrder::NCHW, 0.03f, 17);
        std::shared_ptr<ITensor> weight = std::make_shared<HipTensor>(rt, U8, w.data(), Dim4{16, 1, 3, 3}, DataOrder::NCHW, 0.006f, 140);
        std::shared_ptr<ITensor> bias = std::make_shared<HipTensor>(rt, U8, b.data(), Dim4{1, 16, 1, 1}, DataOrder::NCHW, 0.03f * 0.006f, 0);
        std::shared_ptr<ITensor> output = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{1, 16, 9, 7}, DataOrder::NCHW, 0.02f, 128);
        auto params = std::make_shared<DepthwiseConvolutionParameters>();
        params->padding = {1, 1, 1, 1};
        params->depth_multiplier = 2;
        HipDepthwiseConvolution dw(rt, U8);
        EXPECT(dw.initialize({input, weight, bias}, {output}, params) == Status::SUCCESS);
        EXPECT(input->writeData(x.data()) == Status::SUCCESS);
        EXPECT(dw.execute() == Status::SUCCESS);
        EXPECT(output->readData(got.data()) == Status::SUCCESS);
        EXPECT(same(got, want));
        return ok;
    });

    run_test("FullyConnected.Config2_M256_K4096_N4096", [&] {
        bool ok = true;
        const int m = 256, k = 4096, n = 4096;
        auto a = rand_u8((size_t)m * k, 0xEDE2 + 32);
        std::vector<uint8_t> w((size_t)n * k);
        eo_fill_u8_normal(w.data(), (int64_t)w.size(), 0xEDE2 + 33, 128, 20);
        auto b = rand_i32(n, 0xEDE2 + 34, -1000, 1000);
        eo_quant q;
        eo_make_quant(0.01f, 3, 0.002f, 128, 0.01f * 0.002f, 0.08f, 0, 0, 0, &q);
        EXPECT(q.multiplier == 1099511680 && q.shift == -11);
        std::vector<uint8_t> want((size_t)m * n), got((size_t)m * n);
        eo_fc_u8(a.data(), w.data(), b.data(), want.data(), m, k, n, &q, nullptr);
        std::shared_ptr<ITensor> input = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{(uint32_t)m, (uint32_t)k, 1, 1}, DataOrder::NCHW, 0.01f, 3);
        std::shared_ptr<ITensor> weight = std::make_shared<HipTensor>(rt, U8, w.data(), Dim4{(uint32_t)n, (uint32_t)k, 1, 1}, DataOrder::NCHW, 0.002f, 128);
        std::shared_ptr<ITensor> bias = std::make_shared<HipTensor>(rt, U8, b.data(), Dim4{(uint32_t)n, 1, 1, 1}, DataOrder::NCHW, 0.01f * 0.002f, 0);
        std::shared_ptr<ITensor> output = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{(uint32_t)m, (uint32_t)n, 1, 1}, DataOrder::NCHW, 0.08f, 0);
        HipFullyConnected fc(rt, U8);
        EXPECT(fc.initialize({input, weight, bias}, {output}, std::make_shared<FullyConnectedParameters>()) == Status::SUCCESS);
        EXPECT(input->writeData(a.data()) == Status::SUCCESS);
        EXPECT(fc.execute() == Status::SUCCESS);
        EXPECT(output->readData(got.data()) == Status::SUCCESS);
        EXPECT(same(got, want));
        EXPECT(varied(want));
        EXPECT(fc.release() == Status::SUCCESS);
        return ok;
    });

    run_test("FullyConnected.AndroidNN_flattens_a_4D_input", [&] {
        bool ok = true;
        const int k = 4 * 5 * 6, n = 5;  // input [6][4][5][6] read as 6 rows of 120
        auto a = rand_u8((size_t)6 * k, 61), w = rand_u8((size_t)n * k, 62);
        auto b = rand_i32(n, 63, -100, 100);
        eo_quant q;
        eo_make_quant(0.5f, 100, 0.25f, 90, 0.125f, 40.0f, 128, EO_ACT_RELU1, 1, &q);
        std::vector<uint8_t> want(6 * n), got(6 * n);
        eo_fc_u8(a.data(), w.data(), b.data(), want.data(), 6, k, n, &q, nullptr);
        std::shared_ptr<ITensor> input = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{6, 4, 5, 6}, DataOrder::NCHW, 0.5f, 100);
        std::shared_ptr<ITensor> weight = std::make_shared<HipTensor>(rt, U8, w.data(), Dim4{(uint32_t)n, (uint32_t)k, 1, 1}, DataOrder::NCHW, 0.25f, 90);
        std::shared_ptr<ITensor> bias = std::make_shared<HipTensor>(rt, U8, b.data(), Dim4{(uint32_t)n, 1, 1, 1}, DataOrder::NCHW, 0.125f, 0);
        std::shared_ptr<ITensor> output = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{6, (uint32_t)n, 1, 1}, DataOrder::NCHW, 40.0f, 128);
        auto params = std::make_shared<FullyConnectedParameters>();
        params->androidNN = true;
        params->activation_info = std::make_shared<ActivationInfo>(ActivationInfo::ActivationType::RELU1, true);
        HipFullyConnected fc(rt, U8);
        EXPECT(fc.initialize({input, weight, bias}, {output}, params) == Status::SUCCESS);
        EXPECT(input->writeData(a.data()) == Status::SUCCESS);
        EXPECT(fc.execute() == Status::SUCCESS);
        EXPECT(output->readData(got.data()) == Status::SUCCESS);
        EXPECT(same(got, want));
        return ok;
    });

    run_test("FullyConnected.ReferenceSimpleTest_vector", [&] {
        // src/userdriver/gpu/op_test/fullyconnected_test.cpp:135-149, inputs shifted by a zero point of 10
        bool ok = true;
        const int in_raw[20] = {1, 2, 3, 4, 5, 6, 7, 8, -9, -10, 1, 2, 3, 4, 5, 6, 7, -8, 9, -10};
        std::vector<uint8_t> a(20), w(30);
        for (int i = 0; i < 20; ++i) a[i] = (uint8_t)(in_raw[i] + 10);
        for (int i = 0; i < 30; ++i) w[i] = (uint8_t)(i % 10 + 1);
        std::vector<int32_t> b = {1, 2, 3};
        std::shared_ptr<ITensor> input = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{2, 10, 1, 1}, DataOrder::NCHW, 1.0f, 10);
        std::shared_ptr<ITensor> weight = std::make_shared<HipTensor>(rt, U8, w.data(), Dim4{3, 10, 1, 1}, DataOrder::NCHW, 1.0f, 0);
        std::shared_ptr<ITensor> bias = std::make_shared<HipTensor>(rt, U8, b.data(), Dim4{3, 1, 1, 1}, DataOrder::NCHW, 1.0f, 0);
        std::shared_ptr<ITensor> output = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{2, 3, 1, 1}, DataOrder::NCHW, 1.0f, 0);
        HipFullyConnected fc(rt, U8);
        EXPECT(fc.initialize({input, weight, bias}, {output}, std::make_shared<FullyConnectedParameters>()) == Status::SUCCESS);
        EXPECT(input->writeData(a.data()) == Status::SUCCESS);
        EXPECT(fc.execute() == Status::SUCCESS);
        std::vector<uint8_t> got(6);
        EXPECT(output->readData(got.data()) == Status::SUCCESS);
        const uint8_t expect[6] = {24, 25, 26, 58, 59, 60};
        for (int i = 0; i < 6; ++i) EXPECT(got[i] == expect[i]);
        return ok;
    });

    run_test("Deconvolution.Config4_4x4_stride2_256to128", [&] {
        bool ok = true;
        const eo_conv_shape s = shape(8, 256, 32, 32, 128, 4, 4, 2, 2, 1, 1, 1, 1);
        auto x = rand_u8((size_t)8 * 256 * 1024, 0xEDE2 + 64), w = rand_u8((size_t)256 * 128 * 16, 0xEDE2 + 65);
        auto b = rand_i32(128, 0xEDE2 + 66, -1000, 1000);
        eo_quant q;
        eo_make_quant(0.02f, 121, 0.005f, 133, 0.02f * 0.005f, 0.35f, 128, 0, 0, &q);
        std::vector<uint8_t> want((size_t)8 * 128 * 4096), got(want.size());
        eo_deconv2d_u8(x.data(), w.data(), b.data(), want.data(), &s, &q, nullptr);
        std::shared_ptr<ITensor> input = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{8, 256, 32, 32}, DataOrder::NCHW, 0.02f, 121);
        std::shared_ptr<ITensor> weight = std::make_shared<HipTensor>(rt, U8, w.data(), Dim4{256, 128, 4, 4}, DataOrder::NCHW, 0.005f, 133);
        std::shared_ptr<ITensor> bias = std::make_shared<HipTensor>(rt, U8, b.data(), Dim4{1, 128, 1, 1}, DataOrder::NCHW, 0.02f * 0.005f, 0);
        std::shared_ptr<ITensor> output = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{8, 128, 64, 64}, DataOrder::NCHW, 0.35f, 128);
        auto params = std::make_shared<DeconvolutionParameters>();
        params->padding = {1, 1, 1, 1};
        params->stride = {2, 2};
        HipDeconvolution deconv(rt, U8);
        EXPECT(deconv.initialize({input, weight, bias}, {output}, params) == Status::SUCCESS);
        EXPECT(input->writeData(x.data()) == Status::SUCCESS);
        EXPECT(deconv.execute() == Status::SUCCESS);
        EXPECT(output->readData(got.data()) == Status::SUCCESS);
        EXPECT(same(got, want));
        EXPECT(varied(want));
        EXPECT(deconv.release() == Status::SUCCESS);
        return ok;
    });

    run_test("Deconvolution.AndroidNN_weight_order_channels_last_grouped_planar", [&] {
        bool ok = true;
        {  // androidNN: weight Dim4 = (out, kh, kw, in), channels-last tensors
            const eo_conv_shape s = shape(1, 16, 5, 6, 12, 3, 3, 2, 2, 0, 0, 0, 0);
            const int oh = eo_deconv_out_dim(5, 0, 0, 3, 2), ow = eo_deconv_out_dim(6, 0, 0, 3, 2);
            auto x = rand_u8(16 * 30, 71), w = rand_u8(16 * 12 * 9, 72);  // w in [in][out][kh][kw]
            auto b = rand_i32(12, 73, -100, 100);
            eo_quant q;
            eo_make_quant(0.03f, 131, 0.01f, 77, 0.03f * 0.01f, 0.3f, 5, 0, 0, &q);
            std::vector<uint8_t> want((size_t)12 * oh * ow), got(want.size());
            eo_deconv2d_u8(x.data(), w.data(), b.data(), want.data(), &s, &q, nullptr);
            std::vector<uint8_t> w_nn((size_t)12 * 9 * 16);
            for (int ic = 0; ic < 16; ++ic)
                for (int oc = 0; oc < 12; ++oc)
                    for (int t = 0; t < 9; ++t) w_nn[((size_t)oc * 9 + t) * 16 + ic] = w[((size_t)ic * 12 + oc) * 9 + t];
            std::shared_ptr<ITensor> input = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{1, 5, 6, 16}, DataOrder::NHWC, 0.03f, 131);
            std::shared_ptr<ITensor> weight = std::make_shared<HipTensor>(rt, U8, w_nn.data(), Dim4{12, 3, 3, 16}, DataOrder::NHWC, 0.01f, 77);
            std::shared_ptr<ITensor> bias = std::make_shared<HipTensor>(rt, U8, b.data(), Dim4{1, 12, 1, 1}, DataOrder::NCHW, 0.03f * 0.01f, 0);
            std::shared_ptr<ITensor> output = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{1, (uint32_t)oh, (uint32_t)ow, 12}, DataOrder::NHWC, 0.3f, 5);
            auto params = std::make_shared<DeconvolutionParameters>();
            params->stride = {2, 2};
            params->androidNN = true;
            params->isNCHW = false;
            HipDeconvolution deconv(rt, U8);
            EXPECT(deconv.initialize({input, weight, bias}, {output}, params) == Status::SUCCESS);
            auto x_dev = nchw_to_nhwc(x, 1, 16, 5, 6);
            EXPECT(input->writeData(x_dev.data()) == Status::SUCCESS);
            EXPECT(deconv.execute() == Status::SUCCESS);
            EXPECT(output->readData(got.data()) == Status::SUCCESS);
            EXPECT(same(nhwc_to_nchw(got, 1, 12, oh, ow), want));
        }
        {  // grouped, planar
            const eo_conv_shape s = shape(1, 6, 4, 4, 4, 3, 3, 3, 3, 1, 1, 1, 1, 1, 1, 2);
            const int oh = eo_deconv_out_dim(4, 1, 1, 3, 3);
            auto x = rand_u8(6 * 16, 74), w = rand_u8(6 * 2 * 9, 75);
            auto b = rand_i32(4, 76, -100, 100);
            eo_quant q;
            eo_make_quant(0.03f, 131, 0.01f, 77, 0.03f * 0.01f, 0.1f, 128, 0, 0, &q);
            std::vector<uint8_t> want((size_t)4 * oh * oh), got(want.size());
            eo_deconv2d_u8(x.data(), w.data(), b.data(), want.data(), &s, &q, nullptr);
            std::shared_ptr<ITensor> input = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{1, 6, 4, 4}, DataOrder::NCHW, 0.03f, 131);
            std::shared_ptr<ITensor> weight = std::make_shared<HipTensor>(rt, U8, w.data(), Dim4{6, 2, 3, 3}, DataOrder::NCHW, 0.01f, 77);
            std::shared_ptr<ITensor> bias = std::make_shared<HipTensor>(rt, U8, b.data(), Dim4{1, 4, 1, 1}, DataOrder::NCHW, 0.03f * 0.01f, 0);
            std::shared_ptr<ITensor> output = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{1, 4, (uint32_t)oh, (uint32_t)oh}, DataOrder::NCHW, 0.1f, 128);
            auto params = std::make_shared<DeconvolutionParameters>();
            params->padding = {1, 1, 1, 1};
            params->stride = {3, 3};
            params->group_size = 2;
            HipDeconvolution deconv(rt, U8);
            EXPECT(deconv.initialize({input, weight, bias}, {output}, params) == Status::SUCCESS);
            EXPECT(input->writeData(x.data()) == Status::SUCCESS);
            EXPECT(deconv.execute() == Status::SUCCESS);
            EXPECT(output->readData(got.data()) == Status::SUCCESS);
            EXPECT(same(got, want));
        }
        return ok;
    });

    run_test("Tensor.HostOrderConversion_on_write_and_read", [&] {
        bool ok = true;
        auto x = rand_u8(2 * 5 * 6 * 7, 81);  // planar host data
        HipTensor t(rt, U8, DataType::UINT8, Dim4{2, 5, 6, 7});
        auto x_nhwc = nchw_to_nhwc(x, 2, 5, 6, 7);
        EXPECT(t.writeData(x_nhwc.data(), true, DataOrderChangeType::NHWC2NCHW) == Status::SUCCESS);
        std::vector<uint8_t> got(x.size());
        EXPECT(t.readData(got.data()) == Status::SUCCESS);
        EXPECT(same(got, x));
        EXPECT(t.readData(got.data(), true, DataOrderChangeType::NCHW2NHWC) == Status::SUCCESS);
        EXPECT(same(got, x_nhwc));
        return ok;
    });

    run_test("OperatorList.Pointwise_then_depthwise_over_pooled_buffers", [&] {
        // the block of configuration 3 as an operator list: tensors between operators come from
        // the inter-operator pool and are materialised by assignBufferPool(), as OpenSubGraph does
        bool ok = true;
        const int n = 2;
        auto x = rand_u8((size_t)n * 56 * 56 * 24, 91);  // channels-last
        auto w1 = rand_u8(144 * 24, 92), w2 = rand_u8(144 * 9, 93);
        auto b1 = rand_i32(144, 94, -1000, 1000), b2 = rand_i32(144, 95, -1000, 1000);
        const eo_conv_shape s1 = shape(n, 24, 56, 56, 144, 1, 1), s2 = shape(n, 144, 56, 56, 144, 3, 3, 2, 2, 1, 1, 1, 1);
        eo_quant q1o, q2o;
        eo_make_quant(0.02f, 120, 0.004f, 131, 0.02f * 0.004f, 0.03f, 4, EO_ACT_RELU6, 1, &q1o);
        eo_make_quant(0.03f, 4, 0.006f, 140, 0.03f * 0.006f, 0.025f, 9, EO_ACT_RELU6, 1, &q2o);
        auto x_nchw = nhwc_to_nchw(x, n, 24, 56, 56);
        std::vector<uint8_t> mid((size_t)n * 144 * 56 * 56), want((size_t)n * 144 * 28 * 28), got(want.size());
        eo_conv2d_u8(x_nchw.data(), w1.data(), b1.data(), mid.data(), &s1, &q1o, nullptr);
        eo_dwconv2d_u8(mid.data(), w2.data(), b2.data(), want.data(), &s2, &q2o, nullptr);

        std::shared_ptr<ITensor> in = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{(uint32_t)n, 56, 56, 24}, DataOrder::NHWC, 0.02f, 120, BufferType::INTER_SHARED_NEW);
        std::shared_ptr<ITensor> mid_t = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{(uint32_t)n, 56, 56, 144}, DataOrder::NHWC, 0.03f, 4, BufferType::INTER_SHARED_REUSE);
        std::shared_ptr<ITensor> out = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{(uint32_t)n, 28, 28, 144}, DataOrder::NHWC, 0.025f, 9, BufferType::INTER_SHARED_REUSE);
        auto w1n = nchw_to_nhwc(w1, 144, 24, 1, 1);
        std::shared_ptr<ITensor> w1_t = std::make_shared<HipTensor>(rt, U8, w1n.data(), Dim4{144, 1, 1, 24}, DataOrder::NHWC, 0.004f, 131);
        std::shared_ptr<ITensor> b1_t = std::make_shared<HipTensor>(rt, U8, b1.data(), Dim4{1, 144, 1, 1}, DataOrder::NCHW, 0.02f * 0.004f, 0);
        std::shared_ptr<ITensor> w2_t = std::make_shared<HipTensor>(rt, U8, w2.data(), Dim4{144, 1, 3, 3}, DataOrder::NCHW, 0.006f, 140);
        std::shared_ptr<ITensor> b2_t = std::make_shared<HipTensor>(rt, U8, b2.data(), Dim4{1, 144, 1, 1}, DataOrder::NCHW, 0.03f * 0.006f, 0);
        EXPECT(std::static_pointer_cast<HipTensor>(mid_t)->getDataPtr() == nullptr);  // pooled: not there yet

        auto p1 = std::make_shared<ConvolutionParameters>();
        p1->isNCHW = false;
        p1->activation_info = std::make_shared<ActivationInfo>(ActivationInfo::ActivationType::RELU6, true);
        auto p2 = std::make_shared<DepthwiseConvolutionParameters>();
        p2->isNCHW = false;
        p2->padding = {1, 1, 1, 1};
        p2->stride = {2, 2};
        p2->activation_info = std::make_shared<ActivationInfo>(ActivationInfo::ActivationType::RELU6, true);
        auto conv = std::make_shared<HipConvolution>(rt, U8);
        auto dw = std::make_shared<HipDepthwiseConvolution>(rt, U8);
        EXPECT(conv->initialize({in, w1_t, b1_t}, {mid_t}, p1) == Status::SUCCESS);
        EXPECT(dw->initialize({mid_t, w2_t, b2_t}, {out}, p2) == Status::SUCCESS);
        UDOperators ops = std::make_shared<std::vector<std::shared_ptr<UDOperator>>>();
        ops->push_back(std::make_shared<EnnUDOperator<HipConvolution>>("CONV_2D", 0, UDTensors{in}, UDTensors{mid_t}, UDTensors{w1_t, b1_t}, conv));
        ops->push_back(std::make_shared<EnnUDOperator<HipDepthwiseConvolution>>("DEPTHWISE_CONV_2D", 1, UDTensors{mid_t}, UDTensors{out}, UDTensors{w2_t, b2_t}, dw));
        EXPECT(rt->assignBufferPool() == Status::SUCCESS);
        EXPECT(std::static_pointer_cast<HipTensor>(mid_t)->getDataPtr() != nullptr);
        EXPECT(in->writeData(x.data()) == Status::SUCCESS);
        for (auto &op : *ops) EXPECT(op->execute(nullptr) == ENN_RET_SUCCESS);
        EXPECT(out->readData(got.data()) == Status::SUCCESS);
        EXPECT(same(nhwc_to_nchw(got, n, 144, 28, 28), want));
        for (auto &op : *ops) EXPECT(op->release() == ENN_RET_SUCCESS);
        return ok;
    });

    run_test("Add.Residual_sum_of_two_tensors_with_different_scales", [&] {
        bool ok = true;
        const Dim4 dim = {2, 28, 28, 32};  // channels-last, positional
        const size_t count = (size_t)2 * 28 * 28 * 32;
        auto a = rand_u8(count, 301), b = rand_u8(count, 302);
        std::shared_ptr<ITensor> ta = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, dim, DataOrder::NHWC, 0.0235f, 3);
        std::shared_ptr<ITensor> tb = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, dim, DataOrder::NHWC, 0.011f, 250);
        std::shared_ptr<ITensor> to = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, dim, DataOrder::NHWC, 0.03f, 77);
        auto params = std::make_shared<AddParameters>();
        HipAdd add(rt, U8);
        EXPECT(add.initialize({ta, tb}, {to}, params) == Status::SUCCESS);
        rt->assignBufferPool();
        EXPECT(ta->writeData(a.data()) == Status::SUCCESS);
        EXPECT(tb->writeData(b.data()) == Status::SUCCESS);
        EXPECT(add.execute() == Status::SUCCESS);
        std::vector<uint8_t> got(count), want(count);
        EXPECT(to->readData(got.data()) == Status::SUCCESS);
        eo_add_quant q;
        eo_make_add_quant(0.0235f, 3, 0.011f, 250, 0.03f, 77, 0, 0, &q);
        eo_add_u8(a.data(), b.data(), want.data(), (int64_t)count, &q);
        EXPECT(same(got, want));
        EXPECT(varied(want));
        // a fused ReLU6 narrows the clamp
        params->activation_info = ActivationInfo(ActivationInfo::ActivationType::RELU6, true);
        EXPECT(add.execute() == Status::SUCCESS);
        EXPECT(to->readData(got.data()) == Status::SUCCESS);
        eo_make_add_quant(0.0235f, 3, 0.011f, 250, 0.03f, 77, (int)ActivationInfo::ActivationType::RELU6, 1, &q);
        eo_add_u8(a.data(), b.data(), want.data(), (int64_t)count, &q);
        EXPECT(same(got, want));
        return ok;
    });

    run_test("Averagepool.Global_7x7_channels_last_and_padded_3x3_planar", [&] {
        bool ok = true;
        {
            const int n = 3, c = 1280, h = 7, w = 7;
            auto x = rand_u8((size_t)n * c * h * w, 311);  // planar for the oracle
            std::vector<uint8_t> want((size_t)n * c);
            eo_avgpool_u8(x.data(), want.data(), n, c, h, w, 7, 7, 1, 1, 0, 0, 0, 0, 0, 255);
            std::shared_ptr<ITensor> ti = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{(uint32_t)n, (uint32_t)h, (uint32_t)w, (uint32_t)c}, DataOrder::NHWC, 0.0235f, 0);
            std::shared_ptr<ITensor> to = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{(uint32_t)n, 1, 1, (uint32_t)c}, DataOrder::NHWC, 0.0235f, 0);
            auto params = std::make_shared<Pool2DParameters>();
            params->filter = {7, 7};
            params->isNCHW = false;
            HipAveragepool pool(rt, U8);
            EXPECT(pool.initialize({ti}, {to}, params) == Status::SUCCESS);
            rt->assignBufferPool();
            auto x_nhwc = nchw_to_nhwc(x, n, c, h, w);
            EXPECT(ti->writeData(x_nhwc.data()) == Status::SUCCESS);
            EXPECT(pool.execute() == Status::SUCCESS);
            std::vector<uint8_t> got(want.size());
            EXPECT(to->readData(got.data()) == Status::SUCCESS);
            EXPECT(same(got, want));
            EXPECT(varied(want));
        }
        {
            const int n = 2, c = 5, h = 9, w = 11;
            auto x = rand_u8((size_t)n * c * h * w, 312);
            const int ho = (h + 2 - 3) / 2 + 1, wo = (w + 2 - 3) / 2 + 1;
            std::vector<uint8_t> want((size_t)n * c * ho * wo);
            int32_t lo, hi;
            eo_act_range_u8((int)ActivationInfo::ActivationType::RELU1, 0.01f, 100, &lo, &hi);
            eo_avgpool_u8(x.data(), want.data(), n, c, h, w, 3, 3, 2, 2, 1, 1, 1, 1, lo, hi);
            std::shared_ptr<ITensor> ti = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{(uint32_t)n, (uint32_t)c, (uint32_t)h, (uint32_t)w}, DataOrder::NCHW, 0.01f, 100);
            std::shared_ptr<ITensor> to = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{(uint32_t)n, (uint32_t)c, (uint32_t)ho, (uint32_t)wo}, DataOrder::NCHW, 0.01f, 100);
            auto params = std::make_shared<Pool2DParameters>();
            params->filter = {3, 3};
            params->stride = {2, 2};
            params->padding = {1, 1, 1, 1};
            params->activation_info = ActivationInfo(ActivationInfo::ActivationType::RELU1, true);
            HipAveragepool pool(rt, U8);
            EXPECT(pool.initialize({ti}, {to}, params) == Status::SUCCESS);
            rt->assignBufferPool();
            EXPECT(ti->writeData(x.data()) == Status::SUCCESS);
            EXPECT(pool.execute() == Status::SUCCESS);
            std::vector<uint8_t> got(want.size());
            EXPECT(to->readData(got.data()) == Status::SUCCESS);
            EXPECT(same(got, want));
        }
        return ok;
    });


    // ------------------------------------------------------------ per-channel quantization
    run_test("Convolution.PerChannel_reference_uint8_vector", [&] {
        // src/userdriver/gpu/gpu_userdriver_test.cc:474-576: int8 weights in (out, kh, kw, in) order,
        // one filter scale per output channel, expected output bit for bit
        bool ok = true;
        std::vector<uint8_t> x = {138, 138, 138, 108, 108, 108};
        std::vector<int8_t> w = {1, 2, 1, 2, 1, 2};
        std::vector<int32_t> b = {4, 4, 4};
        const uint8_t expect[9] = {121, 121, 121, 118, 118, 118, 115, 115, 115};
        std::shared_ptr<ITensor> input = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{1, 2, 3, 1}, DataOrder::NCHW, 0.5f, 128);
        std::shared_ptr<ITensor> weight = std::make_shared<HipTensor>(rt, U8, w.data(), Dim4{3, 1, 1, 2}, DataOrder::NCHW, 0.0f, 0);
        std::shared_ptr<ITensor> bias = std::make_shared<HipTensor>(rt, U8, b.data(), Dim4{3, 1, 1, 1});
        std::shared_ptr<ITensor> output = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{1, 3, 3, 1}, DataOrder::NCHW, 1.0f, 128);
        auto params = std::make_shared<ConvolutionParameters>();
        params->androidNN = true;
        params->per_channel_quant = true;
        params->scales = {0.5f, 0.75f, 1.0f};
        HipConvolution conv(rt, U8);
        EXPECT(conv.initialize({input, weight, bias}, {output}, params) == Status::SUCCESS);
        EXPECT(input->writeData(x.data()) == Status::SUCCESS);
        EXPECT(conv.execute() == Status::SUCCESS);
        std::vector<uint8_t> got(9);
        EXPECT(output->readData(got.data()) == Status::SUCCESS);
        for (int i = 0; i < 9; ++i) EXPECT(got[i] == expect[i]);
        return ok;
    });

    // pairs as the per-channel operators derive them: (double)in_scale * (double)filter_scale / (double)out_scale
    auto channel_pairs = [](float s_in, const std::vector<float> &scales, float s_out, std::vector<int32_t> *m, std::vector<int32_t> *sh) {
        m->resize(scales.size());
        sh->resize(scales.size());
        for (size_t i = 0; i < scales.size(); ++i)
            eo_quantize_multiplier((double)s_in * (double)scales[i] / (double)s_out, &(*m)[i], &(*sh)[i]);
    };
    auto channel_scales = [](int count, uint64_t seed, float base) {
        auto r = rand_u8(count, seed);
        std::vector<float> v(count);
        for (int i = 0; i < count; ++i) v[i] = base * (1.0f + 19.0f * r[i] / 255.0f);
        return v;
    };
    auto to_i8 = [](const std::vector<uint8_t> &v) {
        std::vector<int8_t> o(v.size());
        for (size_t i = 0; i < v.size(); ++i) o[i] = (int8_t)((int)v[i] - 128);
        return o;
    };

    run_test("Convolution.PerChannel_channels_last_relu6_and_scales_read_at_execute", [&] {
        bool ok = true;
        const eo_conv_shape s = shape(2, 32, 12, 12, 48, 3, 3, 1, 1, 1, 1, 1, 1);
        auto x = rand_u8((size_t)2 * 32 * 144, 201);
        auto w = to_i8(rand_u8((size_t)48 * 32 * 9, 202));
        auto b = rand_i32(48, 203, -1000, 1000);
        auto scales = channel_scales(48, 204, 0.001f);
        const float s_in = 0.02f, s_out = 0.6f;
        std::vector<int8_t> w_ohwi(w.size());
        for (int o = 0; o < 48; ++o)
            for (int c = 0; c < 32; ++c)
                for (int t = 0; t < 9; ++t) w_ohwi[((size_t)o * 9 + t) * 32 + c] = w[((size_t)o * 32 + c) * 9 + t];
        std::shared_ptr<ITensor> input = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{2, 12, 12, 32}, DataOrder::NHWC, s_in, 117);
        // the filter's own zero point is not used by the per-channel convolution
        std::shared_ptr<ITensor> weight = std::make_shared<HipTensor>(rt, U8, w_ohwi.data(), Dim4{48, 3, 3, 32}, DataOrder::NHWC, 0.0f, 5);
        std::shared_ptr<ITensor> bias = std::make_shared<HipTensor>(rt, U8, b.data(), Dim4{1, 48, 1, 1});
        std::shared_ptr<ITensor> output = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{2, 12, 12, 48}, DataOrder::NHWC, s_out, 20);
        auto params = std::make_shared<ConvolutionParameters>();
        params->padding = {1, 1, 1, 1};
        params->isNCHW = false;
        params->per_channel_quant = true;
        params->scales = scales;
        params->activation_info = std::make_shared<ActivationInfo>(ActivationInfo::ActivationType::RELU6, true);
        HipConvolution conv(rt, U8);
        EXPECT(conv.initialize({input, weight, bias}, {output}, params) == Status::SUCCESS);
        auto x_dev = nchw_to_nhwc(x, 2, 32, 12, 12);
        EXPECT(input->writeData(x_dev.data()) == Status::SUCCESS);
        std::vector<uint8_t> want((size_t)2 * 48 * 144), got(want.size());
        for (int round = 0; round < 2; ++round) {
            if (round == 1)
                for (auto &v : params->scales) v *= 1.7f;  // the next execute() must derive new pairs
            std::vector<int32_t> m, sh;
            channel_pairs(s_in, params->scales, s_out, &m, &sh);
            eo_quant q = {117, 0, 20, 0, 0, 0, 0};
            eo_act_range_u8(EO_ACT_RELU6, s_out, 20, &q.act_min, &q.act_max);
            eo_conv2d_u8_perchannel(x.data(), w.data(), b.data(), want.data(), &s, &q, m.data(), sh.data(), nullptr);
            EXPECT(conv.execute() == Status::SUCCESS);
            EXPECT(output->readData(got.data()) == Status::SUCCESS);
            EXPECT(same(nhwc_to_nchw(got, 2, 48, 12, 12), want));
            EXPECT(varied(want));
        }
        return ok;
    });

    run_test("DepthwiseConvolution.PerChannel_3x3_stride2_channels_last_and_planar_multiplier2", [&] {
        bool ok = true;
        for (int variant = 0; variant < 2; ++variant) {
            const bool nchw = variant == 1;
            const int c = nchw ? 6 : 32, dm = nchw ? 2 : 1, cout = c * dm, h = 13, wdt = 11;
            const eo_conv_shape s = shape(2, c, h, wdt, cout, 3, 3, 2, 2, 1, 1, 1, 1, 1, 1, 1, dm);
            const int ho = eo_conv_out_dim(h, 1, 1, 3, 1, 2), wo = eo_conv_out_dim(wdt, 1, 1, 3, 1, 2);
            auto x = rand_u8((size_t)2 * c * h * wdt, 211 + variant);
            auto w = to_i8(rand_u8((size_t)cout * 9, 213 + variant));
            auto b = rand_i32(cout, 215, -500, 500);
            auto scales = channel_scales(cout, 216, 0.002f);
            const float s_in = 0.02f, s_out = 0.25f;
            std::vector<int32_t> m, sh;
            channel_pairs(s_in, scales, s_out, &m, &sh);
            eo_quant q = {117, -3, 131, 0, 0, 0, 255};  // the filter's zero point is subtracted here
            std::vector<uint8_t> want((size_t)2 * cout * ho * wo), got(want.size());
            eo_dwconv2d_u8_perchannel(x.data(), w.data(), b.data(), want.data(), &s, &q, m.data(), sh.data(), nullptr);
            const DataOrder order = nchw ? DataOrder::NCHW : DataOrder::NHWC;
            Dim4 in_dim = nchw ? Dim4{2, (uint32_t)c, (uint32_t)h, (uint32_t)wdt} : Dim4{2, (uint32_t)h, (uint32_t)wdt, (uint32_t)c};
            Dim4 out_dim = nchw ? Dim4{2, (uint32_t)cout, (uint32_t)ho, (uint32_t)wo} : Dim4{2, (uint32_t)ho, (uint32_t)wo, (uint32_t)cout};
            std::shared_ptr<ITensor> input = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, in_dim, order, s_in, 117);
            std::shared_ptr<ITensor> weight = std::make_shared<HipTensor>(rt, U8, w.data(), Dim4{(uint32_t)cout, 1, 3, 3}, DataOrder::NCHW, 0.0f, -3);
            std::shared_ptr<ITensor> bias = std::make_shared<HipTensor>(rt, U8, b.data(), Dim4{1, (uint32_t)cout, 1, 1});
            std::shared_ptr<ITensor> output = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, out_dim, order, s_out, 131);
            auto params = std::make_shared<DepthwiseConvolutionParameters>();
            params->padding = {1, 1, 1, 1};
            params->stride = {2, 2};
            params->depth_multiplier = dm;
            params->isNCHW = nchw;
            params->per_channel_quant = true;
            params->scales = scales;
            HipDepthwiseConvolution dw(rt, U8);
            EXPECT(dw.initialize({input, weight, bias}, {output}, params) == Status::SUCCESS);
            auto x_dev = nchw ? x : nchw_to_nhwc(x, 2, c, h, wdt);
            EXPECT(input->writeData(x_dev.data()) == Status::SUCCESS);
            EXPECT(dw.execute() == Status::SUCCESS);
            EXPECT(output->readData(got.data()) == Status::SUCCESS);
            EXPECT(same(nchw ? got : nhwc_to_nchw(got, 2, cout, ho, wo), want));
            EXPECT(varied(want));
        }
        return ok;
    });

    run_test("Deconvolution.PerChannel_4x4_stride2_planar_range_derived_for_a_disabled_activation", [&] {
        bool ok = true;
        const eo_conv_shape s = shape(2, 32, 9, 7, 24, 4, 4, 2, 2, 1, 1, 1, 1);
        const int oh = eo_deconv_out_dim(9, 1, 1, 4, 2), ow = eo_deconv_out_dim(7, 1, 1, 4, 2);
        auto x = rand_u8((size_t)2 * 32 * 63, 221);
        auto w = to_i8(rand_u8((size_t)32 * 24 * 16, 222));
        auto b = rand_i32(24, 223, -500, 500);
        auto scales = channel_scales(24, 224, 0.001f);
        const float s_in = 0.02f, s_out = 0.3f;
        std::vector<int32_t> m, sh;
        channel_pairs(s_in, scales, s_out, &m, &sh);
        eo_quant q = {117, 2, 100, 0, 0, 0, 255};
        // CLDeconvolutionPerChannelQuantized.cpp:162-175 derives the range without asking isEnabled()
        eo_act_range_u8(EO_ACT_RELU, s_out, 100, &q.act_min, &q.act_max);
        std::vector<uint8_t> want((size_t)2 * 24 * oh * ow), got(want.size());
        eo_deconv2d_u8_perchannel(x.data(), w.data(), b.data(), want.data(), &s, &q, m.data(), sh.data(), nullptr);
        std::shared_ptr<ITensor> input = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{2, 32, 9, 7}, DataOrder::NCHW, s_in, 117);
        std::shared_ptr<ITensor> weight = std::make_shared<HipTensor>(rt, U8, w.data(), Dim4{32, 24, 4, 4}, DataOrder::NCHW, 0.0f, 2);
        std::shared_ptr<ITensor> bias = std::make_shared<HipTensor>(rt, U8, b.data(), Dim4{1, 24, 1, 1});
        std::shared_ptr<ITensor> output = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{2, 24, (uint32_t)oh, (uint32_t)ow}, DataOrder::NCHW, s_out, 100);
        auto params = std::make_shared<DeconvolutionParameters>();
        params->padding = {1, 1, 1, 1};
        params->stride = {2, 2};
        params->per_channel_quant = true;
        params->scales = scales;
        params->activation_info = std::make_shared<ActivationInfo>(ActivationInfo::ActivationType::RELU, false);
        HipDeconvolution deconv(rt, U8);
        EXPECT(deconv.initialize({input, weight, bias}, {output}, params) == Status::SUCCESS);
        EXPECT(input->writeData(x.data()) == Status::SUCCESS);
        EXPECT(deconv.execute() == Status::SUCCESS);
        EXPECT(output->readData(got.data()) == Status::SUCCESS);
        EXPECT(same(got, want));
        EXPECT(varied(want));
        return ok;
    });

    run_test("PerChannel.ScaleCountAndWeightTypeAreChecked", [&] {
        bool ok = true;
        std::vector<int8_t> w(8 * 8 * 9, 1);
        std::vector<uint8_t> wu(8 * 8 * 9, 1);
        std::vector<int32_t> b(8, 0);
        std::shared_ptr<ITensor> input = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{1, 8, 6, 6}, DataOrder::NCHW, 0.5f, 0);
        std::shared_ptr<ITensor> weight = std::make_shared<HipTensor>(rt, U8, w.data(), Dim4{8, 8, 3, 3});
        std::shared_ptr<ITensor> weight_u8 = std::make_shared<HipTensor>(rt, U8, wu.data(), Dim4{8, 8, 3, 3});
        std::shared_ptr<ITensor> bias = std::make_shared<HipTensor>(rt, U8, b.data(), Dim4{1, 8, 1, 1});
        std::shared_ptr<ITensor> output = std::make_shared<HipTensor>(rt, U8, DataType::UINT8, Dim4{1, 8, 4, 4}, DataOrder::NCHW, 1.0f, 0);
        auto params = std::make_shared<ConvolutionParameters>();
        params->per_channel_quant = true;
        params->scales = std::vector<float>(7, 0.5f);
        HipConvolution short_scales(rt, U8), wrong_type(rt, U8), int8_without_flag(rt, U8);
        EXPECT(short_scales.initialize({input, weight, bias}, {output}, params) == Status::FAILURE);
        params->scales = std::vector<float>(8, 0.5f);
        EXPECT(wrong_type.initialize({input, weight_u8, bias}, {output}, params) == Status::FAILURE);
        EXPECT(int8_without_flag.initialize({input, weight, bias}, {output}, std::make_shared<ConvolutionParameters>()) == Status::FAILURE);
        return ok;
    });


    // ------------------------------------------------------------ INT8 precision
    const PrecisionType S8 = PrecisionType::INT8;
    run_test("Int8.Convolution_channels_last_relu_and_planar_grouped", [&] {
        bool ok = true;
        for (int variant = 0; variant < 2; ++variant) {
            const bool nchw = variant == 1;
            const eo_conv_shape s = nchw ? shape(1, 12, 10, 10, 12, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 3) : shape(2, 32, 12, 12, 48, 3, 3, 2, 2, 1, 1, 1, 1);
            const int cig = s.c / s.groups;
            const int ho = eo_conv_out_dim(s.h, s.pad_t, s.pad_b, s.kh, 1, s.stride_h), wo = eo_conv_out_dim(s.w, s.pad_l, s.pad_r, s.kw, 1, s.stride_w);
            auto x = to_i8(rand_u8((size_t)s.n * s.c * s.h * s.w, 301 + variant));
            auto w = to_i8(rand_u8((size_t)s.cout * cig * 9, 303 + variant));
            auto b = rand_i32(s.cout, 305, -1000, 1000);
            const float s_in = 0.02f, s_w = 0.005f, s_out = 0.2f;
            eo_quant q;
            eo_make_quant_s8(s_in, -9, s_w, 4, s_in * s_w, s_out, -20, EO_ACT_RELU, 1, &q);
            std::vector<int8_t> want((size_t)s.n * s.cout * ho * wo), got(want.size());
            eo_conv2d_s8(x.data(), w.data(), b.data(), want.data(), &s, &q, nullptr, nullptr);
            const DataOrder order = nchw ? DataOrder::NCHW : DataOrder::NHWC;
            Dim4 in_dim = nchw ? Dim4{(uint32_t)s.n, (uint32_t)s.c, (uint32_t)s.h, (uint32_t)s.w} : Dim4{(uint32_t)s.n, (uint32_t)s.h, (uint32_t)s.w, (uint32_t)s.c};
            Dim4 out_dim = nchw ? Dim4{(uint32_t)s.n, (uint32_t)s.cout, (uint32_t)ho, (uint32_t)wo} : Dim4{(uint32_t)s.n, (uint32_t)ho, (uint32_t)wo, (uint32_t)s.cout};
            Dim4 w_dim = nchw ? Dim4{(uint32_t)s.cout, (uint32_t)cig, 3, 3} : Dim4{(uint32_t)s.cout, 3, 3, (uint32_t)cig};
            std::vector<int8_t> w_dev = w;
            if (!nchw)
                for (int o = 0; o < s.cout; ++o)
                    for (int c = 0; c < cig; ++c)
                        for (int t = 0; t < 9; ++t) w_dev[((size_t)o * 9 + t) * cig + c] = w[((size_t)o * cig + c) * 9 + t];
            std::shared_ptr<ITensor> input = std::make_shared<HipTensor>(rt, S8, DataType::INT8, in_dim, order, s_in, -9);
            std::shared_ptr<ITensor> weight = std::make_shared<HipTensor>(rt, S8, w_dev.data(), w_dim, order, s_w, 4);
            std::shared_ptr<ITensor> bias = std::make_shared<HipTensor>(rt, S8, b.data(), Dim4{1, (uint32_t)s.cout, 1, 1}, DataOrder::NCHW, s_in * s_w, 0);
            std::shared_ptr<ITensor> output = std::make_shared<HipTensor>(rt, S8, DataType::INT8, out_dim, order, s_out, -20);
            auto params = std::make_shared<ConvolutionParameters>();
            params->padding = {1, 1, 1, 1};
            params->stride = {(uint32_t)s.stride_h, (uint32_t)s.stride_w};
            params->group_size = s.groups;
            params->isNCHW = nchw;
            params->activation_info = std::make_shared<ActivationInfo>(ActivationInfo::ActivationType::RELU, true);
            HipConvolution conv(rt, S8);
            EXPECT(conv.initialize({input, weight, bias}, {output}, params) == Status::SUCCESS);
            std::vector<int8_t> x_dev = x;
            if (!nchw) {
                auto t = nchw_to_nhwc(std::vector<uint8_t>(x.begin(), x.end()), s.n, s.c, s.h, s.w);
                x_dev.assign(t.begin(), t.end());
            }
            EXPECT(input->writeData(x_dev.data()) == Status::SUCCESS);
            EXPECT(conv.execute() == Status::SUCCESS);
            EXPECT(output->readData(got.data()) == Status::SUCCESS);
            std::vector<uint8_t> g8(got.begin(), got.end()), w8(want.begin(), want.end());
            if (!nchw) g8 = nhwc_to_nchw(g8, s.n, s.cout, ho, wo);
            EXPECT(same(g8, w8));
            EXPECT(varied(w8));
        }
        return ok;
    });

    run_test("Int8.Depthwise_FullyConnected_Deconvolution_Averagepool", [&] {
        bool ok = true;
        const float s_in = 0.02f, s_w = 0.005f;
        {  // depthwise 3x3 stride 1, channels-last
            const int c = 16, h = 9, wd = 10;
            const eo_conv_shape s = shape(2, c, h, wd, c, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1);
            auto x = to_i8(rand_u8((size_t)2 * c * h * wd, 311)), w = to_i8(rand_u8((size_t)c * 9, 312));
            auto b = rand_i32(c, 313, -300, 300);
            eo_quant q;
            eo_make_quant_s8(s_in, 7, s_w, -2, s_in * s_w, 0.05f, -128, EO_ACT_RELU6, 1, &q);
            std::vector<int8_t> want((size_t)2 * c * h * wd), got(want.size());
            eo_dwconv2d_s8(x.data(), w.data(), b.data(), want.data(), &s, &q, nullptr, nullptr);
            std::shared_ptr<ITensor> input = std::make_shared<HipTensor>(rt, S8, DataType::INT8, Dim4{2, (uint32_t)h, (uint32_t)wd, (uint32_t)c}, DataOrder::NHWC, s_in, 7);
            std::shared_ptr<ITensor> weight = std::make_shared<HipTensor>(rt, S8, w.data(), Dim4{(uint32_t)c, 1, 3, 3}, DataOrder::NCHW, s_w, -2);
            std::shared_ptr<ITensor> bias = std::make_shared<HipTensor>(rt, S8, b.data(), Dim4{1, (uint32_t)c, 1, 1}, DataOrder::NCHW, s_in * s_w, 0);
            std::shared_ptr<ITensor> output = std::make_shared<HipTensor>(rt, S8, DataType::INT8, Dim4{2, (uint32_t)h, (uint32_t)wd, (uint32_t)c}, DataOrder::NHWC, 0.05f, -128);
            auto params = std::make_shared<DepthwiseConvolutionParameters>();
            params->padding = {1, 1, 1, 1};
            params->isNCHW = false;
            params->activation_info = std::make_shared<ActivationInfo>(ActivationInfo::ActivationType::RELU6, true);
            HipDepthwiseConvolution dw(rt, S8);
            EXPECT(dw.initialize({input, weight, bias}, {output}, params) == Status::SUCCESS);
            auto t = nchw_to_nhwc(std::vector<uint8_t>(x.begin(), x.end()), 2, c, h, wd);
            EXPECT(input->writeData(t.data()) == Status::SUCCESS);
            EXPECT(dw.execute() == Status::SUCCESS);
            EXPECT(output->readData(got.data()) == Status::SUCCESS);
            EXPECT(same(nhwc_to_nchw(std::vector<uint8_t>(got.begin(), got.end()), 2, c, h, wd), std::vector<uint8_t>(want.begin(), want.end())));
            EXPECT(varied(std::vector<uint8_t>(want.begin(), want.end())));
        }
        {  // fully connected
            const int m = 33, k = 200, n = 70;
            auto a = to_i8(rand_u8((size_t)m * k, 321)), w = to_i8(rand_u8((size_t)n * k, 322));
            auto b = rand_i32(n, 323, -1000, 1000);
            eo_quant q;
            eo_make_quant_s8(s_in, -3, s_w, 0, s_in * s_w, 0.6f, 11, 0, 0, &q);
            std::vector<int8_t> want((size_t)m * n), got(want.size());
            eo_fc_s8(a.data(), w.data(), b.data(), want.data(), m, k, n, &q);
            std::shared_ptr<ITensor> input = std::make_shared<HipTensor>(rt, S8, DataType::INT8, Dim4{(uint32_t)m, (uint32_t)k, 1, 1}, DataOrder::NCHW, s_in, -3);
            std::shared_ptr<ITensor> weight = std::make_shared<HipTensor>(rt, S8, w.data(), Dim4{(uint32_t)n, (uint32_t)k, 1, 1}, DataOrder::NCHW, s_w, 0);
            std::shared_ptr<ITensor> bias = std::make_shared<HipTensor>(rt, S8, b.data(), Dim4{(uint32_t)n, 1, 1, 1}, DataOrder::NCHW, s_in * s_w, 0);
            std::shared_ptr<ITensor> output = std::make_shared<HipTensor>(rt, S8, DataType::INT8, Dim4{(uint32_t)m, (uint32_t)n, 1, 1}, DataOrder::NCHW, 0.6f, 11);
            HipFullyConnected fc(rt, S8);
            EXPECT(fc.initialize({input, weight, bias}, {output}, std::make_shared<FullyConnectedParameters>()) == Status::SUCCESS);
            EXPECT(input->writeData(a.data()) == Status::SUCCESS);
            EXPECT(fc.execute() == Status::SUCCESS);
            EXPECT(output->readData(got.data()) == Status::SUCCESS);
            EXPECT(same(std::vector<uint8_t>(got.begin(), got.end()), std::vector<uint8_t>(want.begin(), want.end())));
            EXPECT(varied(std::vector<uint8_t>(want.begin(), want.end())));
        }
        {  // deconvolution 2x2 stride 2, planar
            const eo_conv_shape s = shape(1, 24, 6, 5, 16, 2, 2, 2, 2);
            auto x = to_i8(rand_u8((size_t)24 * 30, 331)), w = to_i8(rand_u8((size_t)24 * 16 * 4, 332));
            auto b = rand_i32(16, 333, -500, 500);
            eo_quant q;
            eo_make_quant_s8(s_in, 5, s_w, 1, s_in * s_w, 0.12f, -4, 0, 0, &q);
            std::vector<int8_t> want((size_t)16 * 12 * 10), got(want.size());
            eo_deconv2d_s8(x.data(), w.data(), b.data(), want.data(), &s, &q, nullptr, nullptr);
            std::shared_ptr<ITensor> input = std::make_shared<HipTensor>(rt, S8, DataType::INT8, Dim4{1, 24, 6, 5}, DataOrder::NCHW, s_in, 5);
            std::shared_ptr<ITensor> weight = std::make_shared<HipTensor>(rt, S8, w.data(), Dim4{24, 16, 2, 2}, DataOrder::NCHW, s_w, 1);
            std::shared_ptr<ITensor> bias = std::make_shared<HipTensor>(rt, S8, b.data(), Dim4{1, 16, 1, 1}, DataOrder::NCHW, s_in * s_w, 0);
            std::shared_ptr<ITensor> output = std::make_shared<HipTensor>(rt, S8, DataType::INT8, Dim4{1, 16, 12, 10}, DataOrder::NCHW, 0.12f, -4);
            auto params = std::make_shared<DeconvolutionParameters>();
            params->stride = {2, 2};
            HipDeconvolution deconv(rt, S8);
            EXPECT(deconv.initialize({input, weight, bias}, {output}, params) == Status::SUCCESS);
            EXPECT(input->writeData(x.data()) == Status::SUCCESS);
            EXPECT(deconv.execute() == Status::SUCCESS);
            EXPECT(output->readData(got.data()) == Status::SUCCESS);
            EXPECT(same(std::vector<uint8_t>(got.begin(), got.end()), std::vector<uint8_t>(want.begin(), want.end())));
            EXPECT(varied(std::vector<uint8_t>(want.begin(), want.end())));
        }
        {  // average pool 3x3 stride 2 with padding, planar
            auto x = to_i8(rand_u8((size_t)2 * 6 * 9 * 9, 341));
            std::vector<int8_t> want((size_t)2 * 6 * 5 * 5), got(want.size());
            eo_avgpool_s8(x.data(), want.data(), 2, 6, 9, 9, 3, 3, 2, 2, 1, 1, 1, 1, -128, 127);
            std::shared_ptr<ITensor> ti = std::make_shared<HipTensor>(rt, S8, DataType::INT8, Dim4{2, 6, 9, 9}, DataOrder::NCHW, 0.1f, 3);
            std::shared_ptr<ITensor> to = std::make_shared<HipTensor>(rt, S8, DataType::INT8, Dim4{2, 6, 5, 5}, DataOrder::NCHW, 0.1f, 3);
            auto params = std::make_shared<Pool2DParameters>();
            params->padding = {1, 1, 1, 1};
            params->stride = {2, 2};
            params->filter = {3, 3};
            HipAveragepool pool(rt, S8);
            EXPECT(pool.initialize({ti}, {to}, params) == Status::SUCCESS);
            EXPECT(ti->writeData(x.data()) == Status::SUCCESS);
            EXPECT(pool.execute() == Status::SUCCESS);
            EXPECT(to->readData(got.data()) == Status::SUCCESS);
            EXPECT(same(std::vector<uint8_t>(got.begin(), got.end()), std::vector<uint8_t>(want.begin(), want.end())));
        }
        return ok;
    });

    run_test("Int8.TensorTypesMustFitThePrecision", [&] {
        bool ok = true;
        std::vector<uint8_t> wu(8 * 8 * 9, 1);
        std::vector<int32_t> b(8, 0);
        std::shared_ptr<ITensor> input = std::make_shared<HipTensor>(rt, S8, DataType::INT8, Dim4{1, 8, 6, 6}, DataOrder::NCHW, 0.5f, 0);
        std::shared_ptr<ITensor> weight_u8 = std::make_shared<HipTensor>(rt, S8, wu.data(), Dim4{8, 8, 3, 3});
        std::shared_ptr<ITensor> bias = std::make_shared<HipTensor>(rt, S8, b.data(), Dim4{1, 8, 1, 1});
        std::shared_ptr<ITensor> output = std::make_shared<HipTensor>(rt, S8, DataType::INT8, Dim4{1, 8, 4, 4}, DataOrder::NCHW, 1.0f, 0);
        HipConvolution conv(rt, S8);
        EXPECT(conv.initialize({input, weight_u8, bias}, {output}, std::make_shared<ConvolutionParameters>()) == Status::FAILURE);
        HipConvolution fp(rt, PrecisionType::FP16);
        EXPECT(fp.initialize({input, weight_u8, bias}, {output}, std::make_shared<ConvolutionParameters>()) == Status::FAILURE);
        return ok;
    });


    // ------------------------------------------------------------ construction from TFLite options
    auto fmap = [](const char *name, NDims shape, int32_t index, float scale, int32_t zp, TFlite::TensorType type = TFlite::TensorType_UINT8) {
        auto t = std::make_shared<TensorDesc>();
        t->name = name;
        t->shape = shape;
        t->data_type = type;
        t->scale = scale;
        t->zero_point = zp;
        t->buffer_index = index;
        return t;
    };
    auto param = [](const char *name, NDims shape, const void *data, TFlite::TensorType type, float scale, int32_t zp) {
        auto t = std::make_shared<TensorDesc>();
        t->name = name;
        t->shape = shape;
        t->data_type = type;
        t->scale = scale;
        t->zero_point = zp;
        t->is_const = true;
        t->data = data;
        return t;
    };
    auto op_desc = [](const char *name, uint64_t id, TFlite::BuiltinOperator code, std::vector<std::shared_ptr<TensorDesc>> in,
                      std::vector<std::shared_ptr<TensorDesc>> out, std::shared_ptr<void> option) {
        OperatorDesc d;
        d.name = name;
        d.id = id;
        d.code = code;
        d.in_tensors = in;
        d.out_tensors = out;
        d.option = option;
        return d;
    };

    run_test("OpConstructor.AndroidNN_channels_last_residual_network_with_SAME_padding", [&] {
        // input 1x16x16x8 -> conv 3x3 s2 SAME relu6 (16) -> depthwise 3x3 SAME relu6 -> conv 1x1 -> add(conv1) -> pool 8x8 -> fc 10
        bool ok = true;
        const float s0 = 0.02f, sw = 0.004f, s1 = 6.0f / 255, s2 = 6.0f / 255, s3 = 0.05f, s4 = 0.06f, s5 = 0.06f, s6 = 0.1f;
        auto x = rand_u8(16 * 16 * 8, 401);                                  // NHWC
        auto w1 = rand_u8(16 * 9 * 8, 402), wd = rand_u8(9 * 16, 403), w3 = rand_u8(16 * 16, 404), wf = rand_u8(10 * 16, 405);
        auto b1 = rand_i32(16, 406, -500, 500), bd = rand_i32(16, 407, -500, 500), b3 = rand_i32(16, 408, -500, 500), bf = rand_i32(10, 409, -500, 500);
        // ---- oracle, planar
        auto xn = nhwc_to_nchw(x, 1, 8, 16, 16);
        auto w1o = nhwc_to_nchw(w1, 16, 8, 3, 3);                            // [o][kh][kw][i] -> [o][i][kh][kw]
        std::vector<uint8_t> wdo(16 * 9);
        for (int t = 0; t < 9; ++t)
            for (int c = 0; c < 16; ++c) wdo[c * 9 + t] = wd[t * 16 + c];    // [1][kh][kw][c] -> [c][1][kh][kw]
        eo_quant q;
        std::vector<uint8_t> t1(16 * 64), t2(16 * 64), t3(16 * 64), t4(16 * 64), t5(16), want(10), got(10);
        eo_conv_shape c1 = shape(1, 8, 16, 16, 16, 3, 3, 2, 2, 0, 1, 0, 1);  // SAME, TF rule: the extra row and column go last
        eo_make_quant(s0, 128, sw, 120, s0 * sw, s1, 0, EO_ACT_RELU6, 1, &q);
        eo_conv2d_u8(xn.data(), w1o.data(), b1.data(), t1.data(), &c1, &q, nullptr);
        eo_conv_shape c2 = shape(1, 16, 8, 8, 16, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1);
        eo_make_quant(s1, 0, sw, 131, s1 * sw, s2, 0, EO_ACT_RELU6, 1, &q);
        eo_dwconv2d_u8(t1.data(), wdo.data(), bd.data(), t2.data(), &c2, &q, nullptr);
        eo_conv_shape c3 = shape(1, 16, 8, 8, 16, 1, 1);
        eo_make_quant(s2, 0, sw, 125, s2 * sw, s3, 128, 0, 0, &q);
        eo_conv2d_u8(t2.data(), w3.data(), b3.data(), t3.data(), &c3, &q, nullptr);
        eo_add_quant aq;
        eo_make_add_quant(s1, 0, s3, 128, s4, 100, 0, 0, &aq);
        eo_add_u8(t1.data(), t3.data(), t4.data(), 16 * 64, &aq);
        eo_avgpool_u8(t4.data(), t5.data(), 1, 16, 8, 8, 8, 8, 1, 1, 0, 0, 0, 0, 0, 255);
        eo_make_quant(s5, 100, sw, 128, s5 * sw, s6, 128, 0, 0, &q);
        eo_fc_u8(t5.data(), wf.data(), bf.data(), want.data(), 1, 16, 10, &q, nullptr);
        // ---- the list
        const TFlite::TensorType I32 = TFlite::TensorType_INT32, U8T = TFlite::TensorType_UINT8;
        auto f0 = fmap("in", {1, 16, 16, 8}, 0, s0, 128), f1 = fmap("c1", {1, 8, 8, 16}, 1, s1, 0), f2 = fmap("dw", {1, 8, 8, 16}, 2, s2, 0);
        auto f3 = fmap("pw", {1, 8, 8, 16}, 3, s3, 128), f4 = fmap("sum", {1, 8, 8, 16}, 4, s4, 100), f5 = fmap("pool", {1, 1, 1, 16}, 5, s5, 100);
        auto f6 = fmap("logits", {1, 10}, 6, s6, 128);
        auto conv_opt = std::make_shared<TFlite::Conv2DOptions>();
        conv_opt->stride_h = conv_opt->stride_w = 2;
        conv_opt->fused_activation_function = TFlite::ActivationFunctionType_RELU6;
        auto dw_opt = std::make_shared<TFlite::DepthwiseConv2DOptions>();
        dw_opt->fused_activation_function = TFlite::ActivationFunctionType_RELU6;
        auto pw_opt = std::make_shared<TFlite::Conv2DOptions>();
        auto pool_opt = std::make_shared<TFlite::Pool2DOptions>();
        pool_opt->filter_height = pool_opt->filter_width = 8;
        OperatorListDesc list;
        list.legacy_model = TFlite::LegacyModel_ANDROID_NN;
        list.operators = {
            op_desc("CONV_2D", 1, TFlite::BuiltinOperator_CONV_2D,
                    {f0, param("w1", {16, 3, 3, 8}, w1.data(), U8T, sw, 120), param("b1", {16}, b1.data(), I32, s0 * sw, 0)}, {f1}, conv_opt),
            op_desc("DEPTHWISE_CONV_2D", 2, TFlite::BuiltinOperator_DEPTHWISE_CONV_2D,
                    {f1, param("wd", {1, 3, 3, 16}, wd.data(), U8T, sw, 131), param("bd", {16}, bd.data(), I32, s1 * sw, 0)}, {f2}, dw_opt),
            op_desc("CONV_2D", 3, TFlite::BuiltinOperator_CONV_2D,
                    {f2, param("w3", {16, 1, 1, 16}, w3.data(), U8T, sw, 125), param("b3", {16}, b3.data(), I32, s2 * sw, 0)}, {f3}, pw_opt),
            op_desc("ADD", 4, TFlite::BuiltinOperator_ADD, {f1, f3}, {f4}, std::make_shared<TFlite::AddOptions>()),
            op_desc("AVERAGE_POOL_2D", 5, TFlite::BuiltinOperator_AVERAGE_POOL_2D, {f4}, {f5}, pool_opt),
            op_desc("FULLY_CONNECTED", 6, TFlite::BuiltinOperator_FULLY_CONNECTED,
                    {f5, param("wf", {10, 16}, wf.data(), U8T, sw, 128), param("bf", {10}, bf.data(), I32, s5 * sw, 0)}, {f6},
                    std::make_shared<TFlite::FullyConnectedOptions>()),
        };
        for (const int variant : {0, 1, 2}) {  // the Add inside the 1x1 convolution's launch (either operand order), or an operator of its own
            const bool fuse = variant != 2;
            if (variant == 1) {  // the convolution as the Add's first operand: the oracle adds in that order too
                list.operators[3] = op_desc("ADD", 4, TFlite::BuiltinOperator_ADD, {f3, f1}, {f4}, std::make_shared<TFlite::AddOptions>());
                eo_make_add_quant(s3, 128, s1, 0, s4, 100, 0, 0, &aq);
                std::vector<uint8_t> t4b(t4.size());
                eo_add_u8(t3.data(), t1.data(), t4b.data(), 16 * 64, &aq);
                EXPECT(same(t4b, t4));  // the quantized sum does not depend on the operand order
            }
            OperationConstructor built(lib);
            built.fuse_residual_adds = fuse;
            EXPECT(built.open_oplist(list) == ENN_RET_SUCCESS);
            EXPECT(built.operators && built.operators->size() == (fuse ? 5u : 6u));
            EXPECT(built.in_tensors.size() == 1 && built.out_tensors.size() == 1);
            OperationExecutor executor(lib);
            for (int round = 0; round < 2; ++round) {  // a second execution reuses the pooled buffers
                std::fill(got.begin(), got.end(), 0);
                EXPECT(run_list(built, executor, {x.data()}, {got.data()}) == ENN_RET_SUCCESS);
                EXPECT(same(got, want));
            }
            for (auto &o : *built.operators) EXPECT(o->release() == ENN_RET_SUCCESS);
        }
        EXPECT(varied(t4));
        return ok;
    });

    run_test("OpConstructor.Planar_models_Tensorflow_and_Caffe_padding_rules_and_transposed_convolution", [&] {
        bool ok = true;
        const float s0 = 0.02f, sw = 0.004f, s1 = 0.08f, s2 = 0.3f;
        auto x = rand_u8(8 * 15 * 15, 411), w1 = rand_u8(12 * 8 * 9, 412), w2 = rand_u8(12 * 6 * 4, 413);
        auto b1 = rand_i32(12, 414, -500, 500), b2 = rand_i32(6, 415, -500, 500);
        for (int variant = 0; variant < 2; ++variant) {
            const bool caffe = variant == 1;
            // 15 -> 8 with 3x3 stride 2 needs 2 rows of padding: one each side under either rule; 14 -> 7 would differ.
            // Use stride 2 on 15 (symmetric) for the convolution and let the 2x2 stride-2 deconvolution (8 -> 16) follow.
            eo_quant q;
            std::vector<uint8_t> t1(12 * 64), want(6 * 256), got(want.size());
            eo_conv_shape c1 = shape(1, 8, 15, 15, 12, 3, 3, 2, 2, 1, 1, 1, 1);
            eo_make_quant(s0, 128, sw, 120, s0 * sw, s1, 128, 0, 0, &q);
            eo_conv2d_u8(x.data(), w1.data(), b1.data(), t1.data(), &c1, &q, nullptr);
            eo_conv_shape c2 = shape(1, 12, 8, 8, 6, 2, 2, 2, 2);
            eo_make_quant(s1, 128, sw, 130, s1 * sw, s2, 128, EO_ACT_RELU, 1, &q);
            eo_deconv2d_u8(t1.data(), w2.data(), b2.data(), want.data(), &c2, &q, nullptr);
            auto f0 = fmap("in", {1, 8, 15, 15}, 0, s0, 128), f1 = fmap("c1", {1, 12, 8, 8}, 1, s1, 128), f2 = fmap("up", {1, 6, 16, 16}, 2, s2, 128);
            auto conv_opt = std::make_shared<TFlite::Conv2DOptions>();
            conv_opt->stride_h = conv_opt->stride_w = 2;
            auto up_opt = std::make_shared<TFlite::TransposeConvOptions>();
            up_opt->stride_h = up_opt->stride_w = 2;
            up_opt->fused_activation_function = TFlite::ActivationFunctionType_RELU;
            OperatorListDesc list;
            list.legacy_model = caffe ? TFlite::LegacyModel_CAFFE : TFlite::LegacyModel_TENSORFLOW;
            list.operators = {
                op_desc("CONV_2D", 1, TFlite::BuiltinOperator_CONV_2D,
                        {f0, param("w1", {12, 8, 3, 3}, w1.data(), TFlite::TensorType_UINT8, sw, 120),
                         param("b1", {12}, b1.data(), TFlite::TensorType_INT32, s0 * sw, 0)}, {f1}, conv_opt),
                op_desc("TRANSPOSE_CONV", 2, TFlite::BuiltinOperator_TRANSPOSE_CONV,
                        {f1, param("w2", {12, 6, 2, 2}, w2.data(), TFlite::TensorType_UINT8, sw, 130),
                         param("b2", {6}, b2.data(), TFlite::TensorType_INT32, s1 * sw, 0)}, {f2}, up_opt),
            };
            OperationConstructor built(lib);
            EXPECT(built.open_oplist(list) == ENN_RET_SUCCESS);
            OperationExecutor executor(lib);
            EXPECT(run_list(built, executor, {x.data()}, {got.data()}) == ENN_RET_SUCCESS);
            EXPECT(same(got, want));
            EXPECT(varied(want));
        }
        return ok;
    });

    run_test("OpConstructor.Int8_tensors_select_INT8_precision_and_per_channel_scales_select_that_mode", [&] {
        bool ok = true;
        const eo_conv_shape s = shape(1, 16, 9, 9, 24, 3, 3, 1, 1, 1, 1, 1, 1);
        auto x = to_i8(rand_u8(16 * 81, 421)), w = to_i8(rand_u8(24 * 16 * 9, 422));
        auto b = rand_i32(24, 423, -500, 500);
        auto scales = channel_scales(24, 424, 0.002f);
        std::vector<int32_t> m, sh;
        channel_pairs(0.02f, scales, 0.3f, &m, &sh);
        eo_quant q = {-5, 0, 3, 0, 0, -128, 127};
        std::vector<int8_t> want(24 * 81), got(want.size());
        eo_conv2d_s8(x.data(), w.data(), b.data(), want.data(), &s, &q, m.data(), sh.data());
        auto f0 = fmap("in", {1, 16, 9, 9}, 0, 0.02f, -5, TFlite::TensorType_INT8), f1 = fmap("out", {1, 24, 9, 9}, 1, 0.3f, 3, TFlite::TensorType_INT8);
        auto wt = param("w", {24, 16, 3, 3}, w.data(), TFlite::TensorType_INT8, 0.0f, 0);
        wt->per_channel_scales = scales;
        OperatorListDesc list;
        list.legacy_model = TFlite::LegacyModel_TENSORFLOW_NCHW;
        list.operators = {op_desc("CONV_2D", 1, TFlite::BuiltinOperator_CONV_2D, {f0, wt, param("b", {24}, b.data(), TFlite::TensorType_INT32, 1.0f, 0)},
                                  {f1}, std::make_shared<TFlite::Conv2DOptions>())};
        OperationConstructor built(lib);
        EXPECT(built.open_oplist(list) == ENN_RET_SUCCESS);
        OperationExecutor executor(lib);
        EXPECT(run_list(built, executor, {x.data()}, {got.data()}) == ENN_RET_SUCCESS);
        EXPECT(same(std::vector<uint8_t>(got.begin(), got.end()), std::vector<uint8_t>(want.begin(), want.end())));
        EXPECT(varied(std::vector<uint8_t>(want.begin(), want.end())));
        return ok;
    });


    // ------------------------------------------------------------ compute library, executor, userdriver
    run_test("ComputeLibrary.TensorsAndOperatorsComeFromTheLibrary", [&] {
        bool ok = true;
        auto t = lib->create_tensor(TFlite::TensorType_UINT8, U8, NDims{2, 3, 4, 5}, 7, BufferType::DEDICATED, false, StorageType::BUFFER, DataOrder::NCHW, 0.25f, 9);
        EXPECT(t != nullptr);
        if (!t) return false;
        EXPECT(t->getDataType() == DataType::UINT8 && t->getPrecisionType() == U8 && t->getNumOfDims() == 4 && t->getTotalSizeFromDims() == 120);
        EXPECT(t->get_buffer_index() == 7 && t->get_buffer_type() == (uint32_t)TFlite::TensorType_UINT8 && !t->is_const());
        EXPECT(t->getScale() == 0.25f && t->getZeroPoint() == 9);
        auto two = lib->create_tensor(TFlite::TensorType_INT32, U8, NDims{6, 10});   // rank kept, Dim4 padded with ones
        EXPECT(two && two->getNumOfDims() == 2 && two->getDim().h == 1 && two->getDim().w == 1 && two->getNumOfBytes() == 240);
        std::vector<int32_t> b = rand_i32(60, 501, -9999, 9999), back(60);
        DataPtr data = b.data();
        auto c = lib->create_and_copy_tensor(TFlite::TensorType_INT32, data, U8, NDims{60}, UNDEFINED, BufferType::DEDICATED, false, StorageType::BUFFER, DataOrder::NCHW, 0.5f, 0);
        EXPECT(c && c->is_const() && c->getDataType() == DataType::INT32);
        EXPECT(c && c->readData(back.data()) == Status::SUCCESS && back == b);
        auto clone = lib->clone_tensor(t);
        EXPECT(clone && clone->getDims() == t->getDims() && clone->getPrecisionType() == t->getPrecisionType() && clone->get_buffer_index() == 7);
        EXPECT(clone && std::static_pointer_cast<HipTensor>(clone)->getDataPtr() != std::static_pointer_cast<HipTensor>(t)->getDataPtr());
        EXPECT(lib->create_tensor(TFlite::TensorType_UINT8, U8, NDims{1, 1, 2, 2}, UNDEFINED, BufferType::DEDICATED, false, StorageType::TEXTURE) == nullptr);
        EXPECT(lib->create_tensor(TFlite::TensorType_INT64, U8, NDims{4}) == nullptr);
        EXPECT(lib->tensor_type_2_data_type(TFlite::TensorType_INT64) == DataType::SIZE && lib->tensor_type_2_data_type(TFlite::TensorType_INT8) == DataType::INT8);
        EXPECT(lib->setPublicKernels(ANDROID_NN_API, StorageType::BUFFER) == Status::SUCCESS && lib->setPublicKernels(ANDROID_NN_API, StorageType::TEXTURE) == Status::FAILURE);
        // an operator made by the library, on tensors made by the library
        const eo_conv_shape s = shape(1, 16, 9, 9, 24, 3, 3, 1, 1, 1, 1, 1, 1);
        auto x = rand_u8(16 * 81, 502), w = rand_u8(24 * 16 * 9, 503);
        auto bias = rand_i32(24, 504, -500, 500);
        eo_quant q;
        eo_make_quant(0.02f, 128, 0.005f, 120, 0.02f * 0.005f, 0.05f, 3, 0, 0, &q);
        std::vector<uint8_t> want(24 * 81), got(want.size());
        eo_conv2d_u8(x.data(), w.data(), bias.data(), want.data(), &s, &q, nullptr);
        DataPtr wp = w.data(), bp = bias.data();
        auto ti = lib->create_tensor(TFlite::TensorType_UINT8, U8, NDims{1, 16, 9, 9}, 0, BufferType::DEDICATED, false, StorageType::BUFFER, DataOrder::NCHW, 0.02f, 128);
        auto tw = lib->create_and_copy_tensor(TFlite::TensorType_UINT8, wp, U8, NDims{24, 16, 3, 3}, UNDEFINED, BufferType::DEDICATED, false, StorageType::BUFFER, DataOrder::NCHW, 0.005f, 120);
        auto tb = lib->create_and_copy_tensor(TFlite::TensorType_INT32, bp, U8, NDims{24}, UNDEFINED, BufferType::DEDICATED, false, StorageType::BUFFER, DataOrder::NCHW, 0.02f * 0.005f, 0);
        auto to = lib->create_tensor(TFlite::TensorType_UINT8, U8, NDims{1, 24, 9, 9}, 1, BufferType::DEDICATED, false, StorageType::BUFFER, DataOrder::NCHW, 0.05f, 3);
        auto conv = lib->createConvolution(U8);
        auto params = std::make_shared<ConvolutionParameters>();
        params->padding = {1, 1, 1, 1};
        EXPECT(conv->initialize({ti, tw, tb}, {to}, params) == Status::SUCCESS);
        EXPECT(ti->writeData(x.data(), false) == Status::SUCCESS);
        EXPECT(conv->execute() == Status::SUCCESS);
        lib->flush();
        EXPECT(to->readData(got.data(), false) == Status::SUCCESS);   // queued only ...
        lib->synchronize();                                            // ... defined after the library has drained
        EXPECT(same(got, want) && varied(want));
        EXPECT(lib->createAdd(U8) && lib->createAveragepool(U8) && lib->createDeconvolution(U8) && lib->createDepthwiseConvolution(U8) && lib->createFullyConnected(U8));
        return ok;
    });

    run_test("Executor.RecordsOnTheSecondExecutionAndLeavesWeightsAsInputListsAlone", [&] {
        bool ok = true;
        const eo_conv_shape s = shape(2, 8, 10, 10, 16, 3, 3, 1, 1, 1, 1, 1, 1);
        auto x = rand_u8(2 * 8 * 100, 511), w1 = rand_u8(16 * 8 * 9, 512), w2 = rand_u8(16 * 8 * 9, 513);
        auto bias = rand_i32(16, 514, -500, 500);
        eo_quant q;
        eo_make_quant(0.02f, 128, 0.005f, 120, 0.02f * 0.005f, 0.06f, 3, 0, 0, &q);
        std::vector<uint8_t> want1(2 * 16 * 100), want2(want1.size()), got(want1.size());
        eo_conv2d_u8(x.data(), w1.data(), bias.data(), want1.data(), &s, &q, nullptr);
        eo_conv2d_u8(x.data(), w2.data(), bias.data(), want2.data(), &s, &q, nullptr);
        auto conv_opt = std::make_shared<TFlite::Conv2DOptions>();
        for (const bool const_weights : {true, false}) {
            auto f0 = fmap("in", {2, 8, 10, 10}, 0, 0.02f, 128), f1 = fmap("out", {2, 16, 10, 10}, 1, 0.06f, 3);
            auto wt = const_weights ? param("w", {16, 8, 3, 3}, w1.data(), TFlite::TensorType_UINT8, 0.005f, 120) : fmap("w", {16, 8, 3, 3}, 2, 0.005f, 120);
            OperatorListDesc list;
            list.id = const_weights ? 21 : 22;
            list.legacy_model = TFlite::LegacyModel_TENSORFLOW;
            list.operators = {op_desc("CONV_2D", 1, TFlite::BuiltinOperator_CONV_2D, {f0, wt, param("b", {16}, bias.data(), TFlite::TensorType_INT32, 0.02f * 0.005f, 0)}, {f1}, conv_opt)};
            OperationConstructor built(lib);
            EXPECT(built.open_oplist(list) == ENN_RET_SUCCESS);
            EXPECT(built.in_tensors.size() == (const_weights ? 1u : 2u) && built.out_tensors.size() == 1);
            OperationExecutor executor(lib);
            for (int round = 0; round < 4; ++round) {
                std::fill(got.begin(), got.end(), 0);
                const auto &w = round < 2 ? w1 : w2;
                std::vector<const void *> inputs = {x.data()};
                if (!const_weights) inputs.push_back(w.data());
                EXPECT(run_list(built, executor, inputs, {got.data()}) == ENN_RET_SUCCESS);
                EXPECT(same(got, const_weights || round < 2 ? want1 : want2));
            }
            const auto &c = executor.counters();
            if (const_weights)
                EXPECT(c.direct == 1 && c.recordings == 1 && c.replays == 3);
            else
                EXPECT(c.direct == 4 && c.recordings == 0 && c.replays == 0);   // re-packing weights is not replayable
            if (const_weights) {
                // eleven executions in a row on the resident tensors: two bursts of four out of a graph of their own, three single replays
                UDBuffers none;
                BufferTable table;
                std::vector<uint8_t> zeros(got.size(), 0);
                EXPECT(built.out_tensors[0]->writeData(zeros.data()) == Status::SUCCESS);
                EXPECT(executor.execute_times(built.operators, none, table, 11) == ENN_RET_SUCCESS);
                EXPECT(c.direct == 1 && c.recordings == 1 && c.replays == 14);
                EXPECT(built.out_tensors[0]->readData(got.data()) == Status::SUCCESS && same(got, want1));
                // a fresh executor asked for a burst straight away still runs its first execution directly and records at the second
                OperationExecutor second(lib);
                EXPECT(second.execute_times(built.operators, none, table, 6) == ENN_RET_SUCCESS);
                EXPECT(second.counters().direct == 1 && second.counters().recordings == 1 && second.counters().replays == 5);
                EXPECT(built.out_tensors[0]->readData(got.data()) == Status::SUCCESS && same(got, want1));
                second.forget(built.operators);
            }
            executor.forget(built.operators);
            built.close_oplist(list.id);
        }
        EXPECT(varied(want1) && !same(want1, want2));
        return ok;
    });

    run_test("UserDriver.OpenExecuteCloseThroughTheBufferTable", [&] {
        bool ok = true;
        HipUserDriver ud(0);
        EXPECT(ud.Initialize() == ENN_RET_SUCCESS);
        // conv 1x1 (24 -> 48, relu6) -> depthwise 3x3 stride 2 (relu6), channels-last androidNN model
        const float s0 = 0.02f, sw = 0.004f, s1 = 6.0f / 255, s2 = 6.0f / 255;
        auto x = rand_u8(2 * 12 * 12 * 24, 521), w1 = rand_u8(48 * 24, 522), wd = rand_u8(9 * 48, 523);
        auto b1 = rand_i32(48, 524, -500, 500), bd = rand_i32(48, 525, -500, 500);
        auto xn = nhwc_to_nchw(x, 2, 24, 12, 12);
        std::vector<uint8_t> wdo(48 * 9);
        for (int t = 0; t < 9; ++t)
            for (int c = 0; c < 48; ++c) wdo[c * 9 + t] = wd[t * 48 + c];
        eo_quant q;
        std::vector<uint8_t> t1(2 * 48 * 144), t2(2 * 48 * 36);
        eo_conv_shape c1 = shape(2, 24, 12, 12, 48, 1, 1);
        eo_make_quant(s0, 128, sw, 120, s0 * sw, s1, 0, EO_ACT_RELU6, 1, &q);
        eo_conv2d_u8(xn.data(), w1.data(), b1.data(), t1.data(), &c1, &q, nullptr);
        eo_conv_shape c2 = shape(2, 48, 12, 12, 48, 3, 3, 2, 2, 1, 1, 1, 1, 1, 1, 1, 1);
        c2.pad_t = 0; c2.pad_l = 0; c2.pad_b = 1; c2.pad_r = 1;   // SAME at stride 2 on an even extent: the extra row and column go last
        eo_make_quant(s1, 0, sw, 131, s1 * sw, s2, 0, EO_ACT_RELU6, 1, &q);
        eo_dwconv2d_u8(t1.data(), wdo.data(), bd.data(), t2.data(), &c2, &q, nullptr);
        const auto want = nchw_to_nhwc(t2, 2, 48, 6, 6);
        auto f0 = fmap("in", {2, 12, 12, 24}, 10, s0, 128), f1 = fmap("pw", {2, 12, 12, 48}, 11, s1, 0), f2 = fmap("dw", {2, 6, 6, 48}, 12, s2, 0);
        auto pw_opt = std::make_shared<TFlite::Conv2DOptions>();
        pw_opt->fused_activation_function = TFlite::ActivationFunctionType_RELU6;
        auto dw_opt = std::make_shared<TFlite::DepthwiseConv2DOptions>();
        dw_opt->stride_h = dw_opt->stride_w = 2;
        dw_opt->fused_activation_function = TFlite::ActivationFunctionType_RELU6;
        OperatorListDesc list;
        list.id = 0xABCD;
        list.legacy_model = TFlite::LegacyModel_ANDROID_NN;
        list.operators = {
            op_desc("CONV_2D", 1, TFlite::BuiltinOperator_CONV_2D,
                    {f0, param("w1", {48, 1, 1, 24}, w1.data(), TFlite::TensorType_UINT8, sw, 120), param("b1", {48}, b1.data(), TFlite::TensorType_INT32, s0 * sw, 0)}, {f1}, pw_opt),
            op_desc("DEPTHWISE_CONV_2D", 2, TFlite::BuiltinOperator_DEPTHWISE_CONV_2D,
                    {f1, param("wd", {1, 3, 3, 48}, wd.data(), TFlite::TensorType_UINT8, sw, 131), param("bd", {48}, bd.data(), TFlite::TensorType_INT32, s1 * sw, 0)}, {f2}, dw_opt),
        };
        ud.constructor()->fuse_expansions = false;   // this test counts operators: one per description (two images would fuse the pair)
        EXPECT(ud.OpenSubGraph(list) == ENN_RET_SUCCESS);
        EXPECT(ud.OpenSubGraph(list) == ENN_RET_FAILED);   // open already
        EXPECT(ud.PrepareSubGraph(list.id) == ENN_RET_SUCCESS);
        UDOperators ops;
        EXPECT(ud.get_graph_for_TC(list.id, ops) == ENN_RET_SUCCESS && ops && ops->size() == 2 && (*ops)[0]->getName() == "CONV_2D");
        std::vector<uint8_t> got(want.size());
        for (int round = 0; round < 3; ++round) {
            std::fill(got.begin(), got.end(), 0);
            BufferTable table;
            table.add(10, x.data(), x.size());
            table.add(12, got.data(), got.size());
            table.add(99, nullptr, 0);   // an index no tensor of the list has is ignored
            EXPECT(ud.ExecuteSubGraph(OperatorListExecuteRequest(list.id, (uint64_t)round, table)) == ENN_RET_SUCCESS);
            EXPECT(same(got, want));
        }
        EXPECT(ud.executor()->counters().direct == 1 && ud.executor()->counters().recordings == 1 && ud.executor()->counters().replays == 2);
        {
            BufferTable small;
            small.add(10, x.data(), 16);   // too small for the input tensor
            EXPECT(ud.ExecuteSubGraph(OperatorListExecuteRequest(list.id, 9, small)) == ENN_RET_FAILED);
            BufferTable none;
            EXPECT(ud.ExecuteSubGraph(OperatorListExecuteRequest(0x1234, 9, none)) == ENN_RET_FAILED);   // unknown list
        }
        EXPECT(ud.CloseSubGraph(list.id) == ENN_RET_SUCCESS);
        EXPECT(ud.CloseSubGraph(list.id) == ENN_RET_FAILED);
        EXPECT(ud.OpenSubGraph(list) == ENN_RET_SUCCESS);   // and it can be opened again
        EXPECT(ud.CloseSubGraph(list.id) == ENN_RET_SUCCESS);
        // the same list as two lanes of one image each: the list built twice, each lane's operators on its share of the
        // whole input and output tensors, recorded as two branches; then operator by operator on the lanes' streams
        ud.constructor()->image_lanes = 2;
        ud.constructor()->min_lane_images = 1;
        EXPECT(ud.OpenSubGraph(list) == ENN_RET_SUCCESS);
        EXPECT(ud.constructor()->lanes() == 2);
        EXPECT(ud.get_graph_for_TC(list.id, ops) == ENN_RET_SUCCESS && ops && ops->size() == 4);
        if (ops && ops->size() == 4) {
            EXPECT((*ops)[0]->lane() == 0 && (*ops)[1]->lane() == 0 && (*ops)[2]->lane() == 1 && (*ops)[3]->lane() == 1);
            auto in0 = std::static_pointer_cast<HipTensor>((*ops)[0]->getInTensors()[0]), in1 = std::static_pointer_cast<HipTensor>((*ops)[2]->getInTensors()[0]);
            EXPECT(in0->isView() && in1->isView() && in0->getDim().n == 1 && in0->getNumOfBytes() == x.size() / 2);
            EXPECT(static_cast<char *>(in1->getDataPtr()) == static_cast<char *>(in0->getDataPtr()) + x.size() / 2);
            // the lanes' feature maps are different tensors, and the parameters are shared
            EXPECT((*ops)[0]->getOutTensors()[0] != (*ops)[2]->getOutTensors()[0]);
            EXPECT((*ops)[0]->getInTensors()[1] == (*ops)[2]->getInTensors()[1]);
        }
        const auto before = ud.executor()->counters();
        for (int round = 0; round < 5; ++round) {
            if (round == 3) ud.executor()->replay = false;
            std::fill(got.begin(), got.end(), 0);
            BufferTable table;
            table.add(10, x.data(), x.size());
            table.add(12, got.data(), got.size());
            EXPECT(ud.ExecuteSubGraph(OperatorListExecuteRequest(list.id, (uint64_t)round, table)) == ENN_RET_SUCCESS);
            EXPECT(same(got, want));
        }
        ud.executor()->replay = true;
        EXPECT(ud.executor()->counters().direct == before.direct + 3 && ud.executor()->counters().recordings == before.recordings + 1 &&
               ud.executor()->counters().replays == before.replays + 2);
        EXPECT(ud.CloseSubGraph(list.id) == ENN_RET_SUCCESS);
        // three lanes do not divide two images: one chain
        ud.constructor()->image_lanes = 3;
        EXPECT(ud.OpenSubGraph(list) == ENN_RET_SUCCESS && ud.constructor()->lanes() == 1);
        EXPECT(ud.CloseSubGraph(list.id) == ENN_RET_SUCCESS);
        // the pair as one launch, alone and in two lanes: one operator per lane, the expanded tensor without storage,
        // results unchanged
        ud.constructor()->fuse_expansions = true;
        ud.constructor()->fuse_unlisted_expansions = true;
        for (const int lanes : {1, 2}) {
            ud.constructor()->image_lanes = lanes;
            EXPECT(ud.OpenSubGraph(list) == ENN_RET_SUCCESS);
            EXPECT(ud.get_graph_for_TC(list.id, ops) == ENN_RET_SUCCESS && ops && ops->size() == (size_t)lanes);
            if (ops && ops->size() == (size_t)lanes) {
                auto fused = std::dynamic_pointer_cast<EnnUDOperator<HipConvolution>>((*ops)[0]);
                EXPECT(fused && fused->getOp()->hasFusedDepthwise());
                auto expanded = std::static_pointer_cast<HipTensor>((*ops)[0]->getOutTensors()[0]);
                EXPECT(!expanded->hasStorage() && expanded->getDataPtr() == nullptr && expanded->getDim().c == 12);
                EXPECT((*ops)[0]->getOutTensors().size() == 2 && (*ops)[0]->getInTensors().size() == 5);
            }
            for (int round = 0; round < 3; ++round) {
                std::fill(got.begin(), got.end(), 0);
                BufferTable table;
                table.add(10, x.data(), x.size());
                table.add(12, got.data(), got.size());
                EXPECT(ud.ExecuteSubGraph(OperatorListExecuteRequest(list.id, (uint64_t)round, table)) == ENN_RET_SUCCESS);
                EXPECT(same(got, want));
            }
            EXPECT(ud.CloseSubGraph(list.id) == ENN_RET_SUCCESS);
        }
        EXPECT(ud.Deinitialize() == ENN_RET_SUCCESS);
        EXPECT(varied(want));
        return ok;
    });

    std::printf("%d of %d GPU operator tests failed\n", g_failed, g_run);
    return g_failed ? 1 : 0;
}

static int host_tests() {
    // none of these reaches the device: pooled buffers are only sized until assignBufferPool()
    auto rt = std::make_shared<HipRuntime>();
    run_test("BufferPool.InterSharedReuseTakesOverAReleasedBuffer", [&] {
        bool ok = true;
        auto a = rt->getBuffer(U8, DataType::UINT8, Dim4{1, 8, 4, 4}, BufferType::INTER_SHARED_NEW);
        auto b = rt->getBuffer(U8, DataType::UINT8, Dim4{1, 8, 8, 8}, BufferType::INTER_SHARED_REUSE);
        EXPECT(a != b && rt->interPoolSize() == 2);  // nothing released yet: REUSE had to open a new one
        EXPECT(rt->resetInterBuffer(a) == Status::SUCCESS);
        auto c = rt->getBuffer(U8, DataType::UINT8, Dim4{1, 16, 8, 8}, BufferType::INTER_SHARED_REUSE);
        EXPECT(c == a && a->getBytes() == 1024);  // taken over and grown to the larger request
        auto d = rt->getBuffer(U8, DataType::UINT8, Dim4{1, 1, 2, 2}, BufferType::INTER_SHARED_REUSE);
        EXPECT(d != a && d != b && rt->interPoolSize() == 3);
        EXPECT(rt->resetInterBuffer(std::make_shared<HipBuffer>(4)) == Status::FAILURE);
        EXPECT(a->getDataPtr() == nullptr);  // deferred until assignBufferPool
        return ok;
    });
    run_test("BufferPool.ArenasDoNotTakeOverOneAnothersBuffers", [&] {
        bool ok = true;
        auto own = std::make_shared<HipRuntime>();
        auto a = own->getBuffer(U8, DataType::UINT8, Dim4{1, 8, 8, 8}, BufferType::INTER_SHARED_NEW);
        EXPECT(own->resetInterBuffer(a) == Status::SUCCESS);   // free for the next request of its arena
        own->selectArena(1);
        auto b = own->getBuffer(U8, DataType::UINT8, Dim4{1, 8, 4, 4}, BufferType::INTER_SHARED_REUSE);
        EXPECT(b != a && b->arena() == 1 && a->arena() == 0 && own->interPoolSize() == 2);   // another arena: a new buffer
        EXPECT(own->resetInterBuffer(b) == Status::SUCCESS);
        own->selectArena(0);
        auto c = own->getBuffer(U8, DataType::UINT8, Dim4{1, 8, 4, 4}, BufferType::INTER_SHARED_REUSE);
        EXPECT(c == a);                                        // its own arena's free buffer
        own->selectArena(1);
        auto d = own->getBuffer(U8, DataType::UINT8, Dim4{1, 8, 2, 2}, BufferType::INTER_SHARED_REUSE);
        EXPECT(d == b);
        EXPECT(own->abandonPendingBuffers() == Status::SUCCESS && own->interPoolSize() == 0);
        return ok;
    });
    run_test("BufferPool.IntraSharedIsSizedToTheLargestRequest", [&] {
        bool ok = true;
        auto a = rt->getBuffer(U8, DataType::INT32, Dim4{1, 1, 1, 100}, BufferType::INTRA_SHARED);  // 400 B
        auto b = rt->getBuffer(U8, DataType::INT32, Dim4{1, 1, 1, 50}, BufferType::INTRA_SHARED);   // both live: two buffers
        EXPECT(a != b && rt->intraPoolSize() == 2);
        EXPECT(rt->resetIntraBuffer() == Status::SUCCESS);  // next operator
        auto c = rt->getBuffer(U8, DataType::INT32, Dim4{1, 1, 1, 80}, BufferType::INTRA_SHARED);
        EXPECT(c == a);  // the free one that is already large enough
        auto d = rt->getBuffer(U8, DataType::INT32, Dim4{1, 1, 1, 300}, BufferType::INTRA_SHARED);
        EXPECT(d == b && rt->intraPoolSize() == 2);  // the remaining free one, grown to 1200 B
        return ok;
    });
    run_test("Types.LayoutHelpersAndTypeBytes", [&] {
        bool ok = true;
        const Dim4 nhwc = {2, 7, 9, 3};
        const Dim4 nchw = convertDimToNCHW(nhwc);
        EXPECT(nchw.n == 2 && nchw.c == 3 && nchw.h == 7 && nchw.w == 9);
        EXPECT(isDimsSame(convertDimToNHWC(nchw), nhwc));
        EXPECT(getTypeBytes(DataType::UINT8, U8) == 1 && getTypeBytes(DataType::INT32, U8) == 4);
        EXPECT(getTypeBytes(DataType::FLOAT, PrecisionType::FP16) == 2);
        EXPECT(getTensorSizeFromDims(extendToDim4({5, 6})) == 30 && getTensorSizeFromDims(extendToDim4({})) == 0);
        EXPECT(alignTo(1025, 1024) == 2048);
        EXPECT((int)Status::INVALID_PARAMS == 3 && (int)BufferType::INTRA_SHARED == 3 && (int)PrecisionType::UINT8 == 5 &&
               (int)DataType::UINT8 == 4 && (int)DataOrder::NHWC == 1);
        return ok;
    });
    run_test("OpConstructor.PaddingLayoutAndPrecisionRules", [&] {
        bool ok = true;
        typedef OperationConstructor OC;
        Pad4 p;
        // VALID: nothing
        OC::get_padding(TFlite::LegacyModel_TENSORFLOW, TFlite::Padding_VALID, p, {1, 3, 224, 224}, {1, 32, 111, 111}, {32, 3, 3, 3}, {2, 2}, {1, 1}, false, true);
        EXPECT(p.t == 0 && p.b == 0 && p.l == 0 && p.r == 0);
        // SAME, 224 -> 112 with 3x3 stride 2 needs one row: TensorFlow puts it last, Caffe pads both sides with the ceiling
        OC::get_padding(TFlite::LegacyModel_TENSORFLOW, TFlite::Padding_SAME, p, {1, 3, 224, 224}, {1, 32, 112, 112}, {32, 3, 3, 3}, {2, 2}, {1, 1}, false, true);
        EXPECT(p.t == 0 && p.b == 1 && p.l == 0 && p.r == 1);
        OC::get_padding(TFlite::LegacyModel_CAFFE, TFlite::Padding_SAME, p, {1, 3, 224, 224}, {1, 32, 112, 112}, {32, 3, 3, 3}, {2, 2}, {1, 1}, false, true);
        EXPECT(p.t == 1 && p.b == 1 && p.l == 1 && p.r == 1);
        // channels-last extents and (out, kh, kw, in) filters
        OC::get_padding(TFlite::LegacyModel_TENSORFLOW_NHWC, TFlite::Padding_SAME, p, {1, 20, 30, 8}, {1, 20, 30, 16}, {16, 5, 3, 8}, {1, 1}, {1, 1}, false, false);
        EXPECT(p.t == 2 && p.b == 2 && p.l == 1 && p.r == 1);
        // androidNN with planar data still reads the filter as (out, kh, kw, in)
        OC::get_padding(TFlite::LegacyModel_ANDROID_NN, TFlite::Padding_SAME, p, {1, 8, 20, 30}, {1, 16, 20, 30}, {16, 5, 3, 8}, {1, 1}, {1, 1}, false, true);
        EXPECT(p.t == 2 && p.b == 2 && p.l == 1 && p.r == 1);
        // dilation: the reference widens the filter width by dilation.h and the height by dilation.w
        OC::get_padding(TFlite::LegacyModel_TENSORFLOW, TFlite::Padding_SAME, p, {1, 4, 20, 20}, {1, 4, 20, 20}, {4, 4, 3, 3}, {1, 1}, {2, 1}, false, true);
        EXPECT(p.l == 2 && p.r == 2 && p.t == 1 && p.b == 1);
        // transposed convolution: input and output trade places (8 -> 16, 4x4 stride 2 needs 2 in all)
        OC::get_padding(TFlite::LegacyModel_TENSORFLOW, TFlite::Padding_SAME, p, {1, 12, 8, 8}, {1, 6, 16, 16}, {12, 6, 4, 4}, {2, 2}, {1, 1}, true, true);
        EXPECT(p.t == 1 && p.b == 1 && p.l == 1 && p.r == 1);
        // androidNN transposed convolution whose output (18) exceeds (in - 1) * stride + k = 16... no: smaller needed than given -> negative tail
        OC::get_padding(TFlite::LegacyModel_ANDROID_NN, TFlite::Padding_SAME, p, {1, 8, 8, 12}, {1, 18, 18, 6}, {6, 2, 2, 12}, {2, 2}, {1, 1}, true, false);
        EXPECT((int32_t)p.b == -2 && (int32_t)p.r == -2 && p.t == 0 && p.l == 0);
        EXPECT(OC::is_nchw_layout(TFlite::LegacyModel_CAFFE) && OC::is_nchw_layout(TFlite::LegacyModel_TENSORFLOW) &&
               OC::is_nchw_layout(TFlite::LegacyModel_ANDROID_NN) && !OC::is_nchw_layout(TFlite::LegacyModel_TENSORFLOW_NHWC) &&
               !OC::is_nchw_layout(TFlite::LegacyModel_CAFFE_NHWC));
        EXPECT(OC::get_precision(TFlite::TensorType_UINT8) == PrecisionType::UINT8 && OC::get_precision(TFlite::TensorType_INT8) == PrecisionType::INT8 &&
               OC::get_precision(TFlite::TensorType_FLOAT32) == PrecisionType::FP32 && OC::get_precision(TFlite::TensorType_INT32) == PrecisionType::FP16);
        return ok;
    });

    std::printf("%d of %d host-only tests failed\n", g_failed, g_run);
    return g_failed ? 1 : 0;
}

int main(int argc, char **argv) {
    if (argc > 2 && std::strcmp(argv[1], "--filter") == 0) g_filter = argv[2];
    if (argc > 1 && std::strcmp(argv[1], "--host-only") == 0) return host_tests();
    const int rc = host_tests();
    return rc ? rc : gpu_tests();
}
