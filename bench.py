"""Benchmark of the quantized operator hot path on one MI355X.

Headline workload (BASELINE.json configs[1]): uint8 FullyConnected GEMM, M=256
batch rows, K=4096, N=4096, zero points 3 / 128, scales 0.01 / 0.002 / 0.08,
int32 bias, fixed-point requantization fused.  One step = one execution of the
operator on device-resident tensors with pre-packed weights.  The other
configurations are timed the same way and reported under "others"; the
MobileNetV2 figure (BASELINE.json configs[4], the second half of the metric) is
repeated at the top level as "images_per_s".

Memory-bound workloads are timed twice: "warm" replays one set of buffers (every
working set here is smaller than the 256 MB Infinity Cache, so the bytes come
from that cache, not from HBM), "cold" rotates over enough buffer sets that a
set has been evicted before it is used again.  For the HBM-bound workloads
under "others" the cold figure is the one the roofline fraction is quoted on
(the warm one stands beside it as roofline_warm).  The headline (`value`,
`roofline`) is the warm figure of the MFMA-bound GEMM; its cold figure stands at
the top level as `roofline_cold`.

The MobileNetV2 figure is given twice: `images_per_s` (operator plans over the
C ABI, one graph replay per four batches) and `images_per_s_operator_api` (the
network described as an operator list, built by the C++ OperationConstructor and
run by the OperationExecutor, the level the reference binds its userdriver at).

Prints ONE JSON line.  `--gpus N` with N > 1 is refused: this build uses one GPU."""
import argparse
import importlib
import json
import os
import re
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

INT8_PEAK_TOPS = 5000.0   # MI355X dense int8 MFMA peak, TOP/s
HBM_PEAK_GBS = 8000.0     # MI355X HBM3E peak, GB/s
SEED = 0xEDE2
COLD_FOOTPRINT = 640 << 20   # bytes a rotating workload walks through before it comes back: 2.5 x the Infinity Cache
HEADLINE_PROFILE = os.path.join(ROOT, "profiles", "igemm_dma_64x64_splitk__fc_m256_k4096_n4096.md")
CLOCK_RAMP_SECONDS = 0.5   # untimed work before the first timed region of the process
_clocks_ramped = False
MIN_TIMED_SECONDS = 0.02   # a timed region shorter than this is mostly host overhead: the K steps are then repeated


def time_steps(eden, stream, launch, steps, warmup, use_graph=True, chunk=50, sets=1):
    """Runs `warmup` untimed and `steps` timed executions of launch(stream_handle, set_index), set_index walking
    0 .. sets-1 round and round (workloads that rotate over several buffer sets to defeat the caches).  When the K
    steps take less than MIN_TIMED_SECONDS the whole K-step region is repeated R times inside the timed region.
    Returns (wall seconds per K steps, HIP-event seconds per K steps, R)."""
    counter = [0]

    def one(s):
        launch(s, counter[0] % sets)
        counter[0] += 1

    for _ in range(max(warmup, sets)):
        one(stream.h)
    stream.sync()
    graph = None
    chunk = max(1, min(chunk, steps))
    if sets > 1:
        chunk = max(sets, chunk // sets * sets)  # a replay walks whole rounds of the buffer sets
        steps = -(-steps // chunk) * chunk if use_graph else steps  # (callers pass whole rounds: see round_steps)
    if use_graph and chunk <= steps:
        counter[0] = 0
        graph = eden.Graph(stream, lambda s: [one(s) for _ in range(chunk)])
        graph.launch(stream)  # first replay uploads the graph; keep it out of the timed region
        stream.sync()

    def region():
        done = 0
        if graph is not None:
            while done + chunk <= steps:
                graph.launch(stream)
                done += chunk
        while done < steps:
            one(stream.h)
            done += 1

    # The first workload of a process meets a GPU that may have idled at its lowest clocks (a fresh machine takes some
    # tenths of a second of work to leave them): half a second of untimed replays of the same region comes first.
    global _clocks_ramped
    if not _clocks_ramped:
        _clocks_ramped = True
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < CLOCK_RAMP_SECONDS:
            region()
            stream.sync()
    e0, e1 = eden.Event(), eden.Event()
    repeats, wall, ev = 1, 0.0, 0.0
    while True:
        device_sync()
        t0 = time.perf_counter()
        e0.record(stream.h)
        for _ in range(repeats):
            region()
        e1.record(stream.h)
        stream.sync()
        device_sync()
        wall = time.perf_counter() - t0
        ev = e1.elapsed_ms_since(e0) * 1e-3
        if wall >= MIN_TIMED_SECONDS or repeats >= 4096:
            break
        repeats = min(4096, max(repeats * 2, int(repeats * MIN_TIMED_SECONDS * 1.3 / max(wall, 1e-6)) + 1))
    return wall / repeats, ev / repeats, repeats


_torch = None


def device_sync():
    """torch.cuda.synchronize() when torch is importable (device-wide), plus the library's own sync."""
    global _torch
    if _torch is None:
        try:
            import torch
            _torch = torch if torch.cuda.is_available() else False
        except Exception:
            _torch = False
    if _torch:
        _torch.cuda.synchronize()
    eden_mod.sync(None)


def round_steps(steps, sets, chunk=50):
    """`steps` rounded up to whole graph replays of a rotating workload, so that no launch of the timed region comes from the host"""
    if sets <= 1:
        return steps
    chunk = max(sets, min(chunk, steps) // sets * sets)
    return -(-steps // chunk) * chunk


def set_count(per_set_bytes, cold):
    return max(2, -(-COLD_FOOTPRINT // per_set_bytes)) if cold else 1


def fc_workload(eden, synth, m=256, k=4096, n=4096, cold=False):
    """cold: every set has its own activations, weights (packed per plan) and output"""
    a = synth.fill_u8((m, k), SEED + 32)
    w = synth.fill_u8_normal((n, k), SEED + 33, 128, 20)
    b = synth.fill_i32((n,), SEED + 34, -1000, 1000)
    q = eden.make_requant(0.01, 3, 0.002, 128, 0.08, 0)
    nbytes = m * k + n * k + 4 * n + m * n
    sets = set_count(nbytes, cold)
    d_b = eden.DeviceBuffer(host=b)
    per_set = []
    for _ in range(sets):
        d_a, d_w, d_o = eden.DeviceBuffer(host=a), eden.DeviceBuffer(host=w), eden.DeviceBuffer(nbytes=m * n)
        plan = eden.FcPlan(m, k, n, d_w, d_b, q)
        if cold:
            eden.sync()
            d_w.free()   # the plan keeps its own packed copy; the raw weights are not read again
        per_set.append((d_a, d_o, plan))
    return dict(name="fc_m%d_k%d_n%d" % (m, k, n), launch=lambda s, i: per_set[i][2].run(per_set[i][0], per_set[i][1], q, s),
                keep=(per_set, d_b), sets=sets, ops=2.0 * m * k * n, bytes=nbytes,
                # (few rows: the weights' trip from HBM is the lower roof; the published peaks meet at 625 operations per byte)
                bound="mfma" if m >= 256 or 2.0 * m * k * n / nbytes >= 625 else "hbm",
                host=(a, w, b, q), out=per_set[0][1], out_shape=(m, n))


def conv_workload(eden, synth, n=1, cold=False, cin=64, cout=64, hw=56, k=3, stride=1, dil=1):
    """k x k convolution, ReLU, channels-last: BASELINE configs[0] (3x3, 64 -> 64 channels at 56 x 56) by default"""
    pad = dil * (k - 1) // 2
    ho = (hw + 2 * pad - dil * (k - 1) - 1) // stride + 1
    desc = eden.conv_desc(n, cin, hw, hw, cout, k, k, stride=(stride, stride), pad=(pad,) * 4, dil=(dil, dil), layout=eden.NHWC)
    x = synth.fill_u8((n, hw, hw, cin), SEED + 16)
    w = synth.fill_u8((cout, cin, k, k), SEED + 17)
    b = synth.fill_i32((cout,), SEED + 18, -1000, 1000)
    q = eden.make_requant(0.02, 128, 0.005, 120, 0.05 * (cin * k * k / 576.0) ** 0.5, 0, eden.ACT_RELU, True)
    d_w, d_b = eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
    plan = eden.ConvPlan(desc, d_w, d_b, q)
    nbytes = n * hw * hw * cin + n * ho * ho * cout + cout * cin * k * k + 4 * cout
    sets = set_count(nbytes, cold)
    bufs = [(eden.DeviceBuffer(host=x), eden.DeviceBuffer(nbytes=n * ho * ho * cout)) for _ in range(sets)]
    name = "conv3x3_n%d_c64_56x56_nhwc" % n if (cin, cout, hw, k, stride) == (64, 64, 56, 3, 1) else \
        "conv%dx%ds%d%s_n%d_%dto%d_%dx%d_nhwc" % (k, k, stride, "" if dil == 1 else "d%d" % dil, n, cin, cout, hw, hw)
    return dict(name=name, launch=lambda s, i: plan.run(bufs[i][0], bufs[i][1], q, s),
                keep=(bufs, d_w, d_b, plan), sets=sets, ops=2.0 * n * ho * ho * cout * cin * k * k, bytes=nbytes,
                # (which roof is the lower one: the published peaks meet at 5000 / 8 = 625 operations per byte)
                bound="mfma" if (cin, cout, hw, k, stride) == (64, 64, 56, 3, 1) or 2.0 * n * ho * ho * cout * cin * k * k / nbytes >= 625 else "hbm")


def dw_workload(eden, synth, n=32, cold=False, c=144, hw=56, stride=2, k=3, dil=1):
    """depthwise k x k convolution, ReLU6, channels-last: BASELINE configs[2]'s stride-2 3x3 layer by default"""
    pad = dil * (k - 1) // 2
    ho = (hw + 2 * pad - dil * (k - 1) - 1) // stride + 1
    desc = eden.conv_desc(n, c, hw, hw, c, k, k, stride=(stride, stride), pad=(pad,) * 4, dil=(dil, dil), dm=1, layout=eden.NHWC)
    x = synth.fill_u8((n, hw, hw, c), SEED + 48)
    w = synth.fill_u8((c, 1, k, k), SEED + 49)
    b = synth.fill_i32((c,), SEED + 50, -1000, 1000)
    q = eden.make_requant(0.03, 17, 0.006, 140, 0.025 * k / 3, 9, eden.ACT_RELU6, True)
    d_w, d_b = eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
    plan = eden.DwConvPlan(desc, d_w, d_b, q)
    nbytes = n * c * hw * hw + c * k * k + c * 4 + n * c * ho * ho
    sets = set_count(nbytes, cold)
    bufs = [(eden.DeviceBuffer(host=x), eden.DeviceBuffer(nbytes=n * ho * ho * c)) for _ in range(sets)]
    return dict(name="dw%dx%ds%d%s_n%d_c%d_%dx%d_nhwc" % (k, k, stride, "" if dil == 1 else "d%d" % dil, n, c, hw, hw), launch=lambda s, i: plan.run(bufs[i][0], bufs[i][1], q, s),
                keep=(bufs, d_w, d_b, plan), sets=sets, ops=2.0 * n * c * ho * ho * k * k, bytes=nbytes, bound="hbm")


def pw_workload(eden, synth, n=32, cin=24, cout=144, hw=56, cold=False):
    """pointwise (1x1) convolution, ReLU6: BASELINE configs[2]'s expansion by default; (64, 384, 14) and (384, 64, 14) are the
    expansion and projection of MobileNetV2's 14x14 stage"""
    if (cin, cout, hw) != (24, 144, 56):
        desc = eden.conv_desc(n, cin, hw, hw, cout, 1, 1, layout=eden.NHWC)
        x = synth.fill_u8((n, hw, hw, cin), SEED + 51)
        w = synth.fill_u8_normal((cout, cin, 1, 1), SEED + 52, 128, 40)
        b = synth.fill_i32((cout,), SEED + 53, -1000, 1000)
        q = eden.make_requant(0.02, 120, 0.004, 131, 0.03 * (cin / 24) ** 0.5, 4, eden.ACT_RELU6, True)
        d_w, d_b = eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
        plan = eden.ConvPlan(desc, d_w, d_b, q)
        nbytes = n * hw * hw * cin + cout * cin + 4 * cout + n * hw * hw * cout
        sets = set_count(nbytes, cold)
        bufs = [(eden.DeviceBuffer(host=x), eden.DeviceBuffer(nbytes=n * hw * hw * cout)) for _ in range(sets)]
        return dict(name="pw1x1_n%d_%dto%d_%dx%d_nhwc" % (n, cin, cout, hw, hw), launch=lambda s, i: plan.run(bufs[i][0], bufs[i][1], q, s),
                    keep=(bufs, d_w, d_b, plan), sets=sets, ops=2.0 * n * hw * hw * cin * cout, bytes=nbytes, bound="hbm")
    desc = eden.conv_desc(n, 24, 56, 56, 144, 1, 1, layout=eden.NHWC)
    x = synth.fill_u8((n, 56, 56, 24), SEED + 51)
    w = synth.fill_u8((144, 24, 1, 1), SEED + 52)
    b = synth.fill_i32((144,), SEED + 53, -1000, 1000)
    q = eden.make_requant(0.02, 120, 0.004, 131, 0.03, 4, eden.ACT_RELU6, True)
    d_w, d_b = eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
    plan = eden.ConvPlan(desc, d_w, d_b, q)
    nbytes = n * 56 * 56 * 24 + 144 * 24 + 576 + n * 56 * 56 * 144
    sets = set_count(nbytes, cold)
    bufs = [(eden.DeviceBuffer(host=x), eden.DeviceBuffer(nbytes=n * 56 * 56 * 144)) for _ in range(sets)]
    return dict(name="pw1x1_n%d_24to144_56x56_nhwc" % n, launch=lambda s, i: plan.run(bufs[i][0], bufs[i][1], q, s),
                keep=(bufs, d_w, d_b, plan), sets=sets, ops=2.0 * n * 56 * 56 * 24 * 144, bytes=nbytes, bound="hbm")


def block_workload(eden, synth, n=32, rows=0, cols=0, cold=False, cin=24, c=144, hw=56, stride=2, fused=True):
    """A pointwise expansion cin -> c (ReLU6) feeding a 3x3 depthwise convolution.  fused: one launch, the expanded
    tensor held in LDS (eh_conv_dw_block_run); otherwise the two stand-alone launches with the expanded tensor in
    device memory.  The default shape is BASELINE configs[2].  Algorithmic bytes = the block's input, weights and
    output either way (the expanded tensor is an intermediate)."""
    ho = (hw + 2 - 3) // stride + 1
    d1 = eden.conv_desc(n, cin, hw, hw, c, 1, 1, layout=eden.NHWC)
    d2 = eden.conv_desc(n, c, hw, hw, c, 3, 3, stride=(stride, stride), pad=(1, 1, 1, 1), dm=1, layout=eden.NHWC)
    x = synth.fill_u8((n, hw, hw, cin), SEED + 51)
    w1, b1 = synth.fill_u8((c, cin, 1, 1), SEED + 52), synth.fill_i32((c,), SEED + 53, -1000, 1000)
    w2, b2 = synth.fill_u8((c, 1, 3, 3), SEED + 49), synth.fill_i32((c,), SEED + 50, -1000, 1000)
    q1 = eden.make_requant(0.02, 120, 0.004, 131, 0.03, 17, eden.ACT_RELU6, True)
    q2 = eden.make_requant(0.03, 17, 0.006, 140, 0.025, 9, eden.ACT_RELU6, True)
    keep = [eden.DeviceBuffer(host=a) for a in (w1, b1, w2, b2)]
    pw, dw = eden.ConvPlan(d1, keep[0], keep[1], q1), eden.DwConvPlan(d2, keep[2], keep[3], q2)
    nbytes = n * hw * hw * cin + c * cin + 4 * c + c * 9 + 4 * c + n * ho * ho * c
    sets = set_count(nbytes + (0 if fused else 2 * n * hw * hw * c), cold)
    bufs = [(eden.DeviceBuffer(host=x), eden.DeviceBuffer(nbytes=n * ho * ho * c)) for _ in range(sets)]
    if fused:
        assert eden.conv_dw_block_applies(pw, dw)
        launch = lambda s, i: eden.conv_dw_block_run(pw, dw, bufs[i][0], bufs[i][1], q1, q2, rows, cols, stream=s)
    else:
        mids = [eden.DeviceBuffer(nbytes=n * hw * hw * c) for _ in range(sets)]
        keep.append(mids)

        def launch(s, i):
            pw.run(bufs[i][0], mids[i], q1, s)
            dw.run(mids[i], bufs[i][1], q2, s)
    shape = "c3block_n%d" % n if (cin, c, hw, stride) == (24, 144, 56, 2) else "block_n%d" % n
    return dict(name="%s_pw%dto%d_dw3x3s%d_%dx%d_nhwc%s%s" % (shape, cin, c, stride, hw, hw, "" if fused else "_two_launches",
                                                             "_tile%dx%d" % (rows, cols) if rows or cols else ""),
                launch=launch, keep=(bufs, keep, pw, dw), sets=sets, ops=2.0 * n * (hw * hw * cin * c + ho * ho * c * 9), bytes=nbytes, bound="hbm")


def deconv_workload(eden, synth, n=8, cold=False, cin=256, cout=128, hw=32, k=4, stride=2):
    """transposed convolution, channels-last: BASELINE configs[3] (4x4 stride 2, 256 -> 128 channels at 32 x 32) by default"""
    pad = (k - stride) // 2 if k >= stride else 0
    ho = (hw - 1) * stride + k - 2 * pad
    desc = eden.conv_desc(n, cin, hw, hw, cout, k, k, stride=(stride, stride), pad=(pad,) * 4, layout=eden.NHWC,
                          weight_layout=eden.W_IOHW)
    x = synth.fill_u8((n, hw, hw, cin), SEED + 64)
    w = synth.fill_u8((cin, cout, k, k), SEED + 65)
    b = synth.fill_i32((cout,), SEED + 66, -1000, 1000)
    q = eden.make_requant(0.02, 121, 0.005, 133, 0.35 * (cin * k * k / 4096.0) ** 0.5, 128)
    d_w, d_b = eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
    plan = eden.DeconvPlan(desc, d_w, d_b, q)
    nbytes = n * cin * hw * hw + cin * cout * k * k + 4 * cout + n * cout * ho * ho
    sets = set_count(nbytes, cold)
    bufs = [(eden.DeviceBuffer(host=x), eden.DeviceBuffer(nbytes=n * ho * ho * cout)) for _ in range(sets)]
    ops = 2.0 * n * hw * hw * cin * cout * k * k   # every input pixel meets every tap once
    return dict(name="deconv%dx%ds%d_n%d_%dto%d_%dx%d_nhwc" % (k, k, stride, n, cin, cout, hw, hw), launch=lambda s, i: plan.run(bufs[i][0], bufs[i][1], q, s),
                keep=(bufs, d_w, d_b, plan), sets=sets, ops=ops, bytes=nbytes,
                bound="mfma" if (cin, cout, hw, k, stride) == (256, 128, 32, 4, 2) or ops / nbytes >= 625 else "hbm")


def mbv2_workload(eden, synth, batch=64, per_channel=False, weights="minmax", cold=False, lanes=2, fuse_blocks="auto"):
    """BASELINE.json configs[4]: MobileNetV2-1.0 uint8 at 224x224x3, batch 64, the whole operator list per step,
    its feature maps in the library's buffer pool (liveness reuse as the reference's operator constructor does it, one
    device allocation; the network input keeps its own slot, so every step reads the same images).
    weights: "minmax" = per-tensor min/max quantized random-init weights (bytes span 0 .. 255), the configuration
    BASELINE.json names; "narrow" = N(zp, 20) bytes.  per_channel: int8 weights with one scale per output channel in
    the convolutions.  A step streams every feature map once, more than the Infinity Cache holds (working_set).
    lanes: the step's images run as that many independent chains of batch / lanes images on streams of their own
    (parallel branches of the replayed graph; 1 = one chain of full-batch launches).  fuse_blocks: "auto" runs the
    expansion + depthwise pairs the library's measured table prefers as one launch each, () none."""
    mobilenet = importlib.import_module("cl-eden-kernel_amd.mobilenet")
    # residual adds inside the projection convolutions' launches
    net = mobilenet.MobileNetV2(eden, batch, fuse_add=True, per_channel=per_channel, weights=weights, pooled=True, lanes=lanes,
                                fuse_blocks=fuse_blocks)
    net.set_input(mobilenet.network_input(batch))
    name = "mobilenet_v2_1.0_224_u8%s%s_batch%d%s%s" % ("_perchannel_w" if per_channel else "", "" if weights == "minmax" else "_narrow_w", batch,
                                                       "_%dlanes" % net.lanes if net.lanes > 1 else "",
                                                       "_%dfused_blocks" % len(net.fused_blocks) if net.fused_blocks else "")
    return dict(name=name, launch=lambda s, i: net.run(s), keep=net, sets=1, net=net,
                ops=2.0 * mobilenet.macs_per_image() * batch, bytes=mobilenet.compulsory_bytes_per_image() * batch,
                bound="hbm", images=batch, chunk=4, per_channel=per_channel, weights=weights,
                working_set=sum(batch * t["h"] * t["w"] * t["c"] for i, t in enumerate(net.tensors) if i not in net.unwritten and i not in net.in_lds),
                pool_bytes=net.pool_bytes, lanes=net.lanes, fused_blocks=list(net.fused_blocks))


def mbv2_userdriver(eden, batch=64, per_channel=False, list_id=0xC5, planar=False):
    """The same network through the operator API the reference binds: described as an operator list, opened by the C++
    OperationConstructor on a HipComputeLibrary (HipConvolution ... operators, pooled feature maps), executed by the
    OperationExecutor, which records the list into a HIP graph on its second execution and replays it.  Returns
    (driver, list id, logits shape); the input tensor holds network_input(batch).  planar: the model as a planar list
    (feature maps [n, c, h, w]), whose feature maps the constructor stores channels-last behind one layout operator."""
    mobilenet = importlib.import_module("cl-eden-kernel_amd.mobilenet")
    ud = importlib.import_module("cl-eden-kernel_amd.userdriver")
    driver = ud.UserDriver(0)
    ol, _, _, shape = mobilenet.operator_list(ud, list_id, batch, per_channel=per_channel, nchw=planar)
    driver.open_subgraph(ol)
    x = mobilenet.network_input(batch)
    driver.write_input(list_id, 0, np.ascontiguousarray(x.transpose(0, 3, 1, 2)) if planar else x)
    return driver, list_id, shape


def time_userdriver(eden, driver, list_id, steps, warmup):
    """`steps` executions of the list's operators (OperationExecutor::execute, tensors resident), timed by wall clock
    and by HIP events on the userdriver's own stream; repeated like time_steps when shorter than MIN_TIMED_SECONDS."""
    driver.execute_operators(list_id, max(warmup, 3))   # the first runs operator by operator, the second records
    driver.synchronize()
    e0, e1 = eden.Event(), eden.Event()
    repeats = 1
    while True:
        device_sync()
        t0 = time.perf_counter()
        e0.record(driver.stream)
        driver.execute_operators(list_id, steps * repeats)
        e1.record(driver.stream)
        driver.synchronize()
        device_sync()
        wall = time.perf_counter() - t0
        ev = e1.elapsed_ms_since(e0) * 1e-3
        if wall >= MIN_TIMED_SECONDS or repeats >= 4096:
            return wall / repeats, ev / repeats, repeats
        repeats = min(4096, max(repeats * 2, int(repeats * MIN_TIMED_SECONDS * 1.3 / max(wall, 1e-6)) + 1))


def copy_workload(eden, synth, mib=64, cold=False):
    """A plain device-to-device copy of known size: the yardstick the HBM byte counters are scaled by."""
    nbytes = mib << 20
    sets = set_count(2 * nbytes, cold)
    bufs = [(eden.DeviceBuffer(nbytes=nbytes), eden.DeviceBuffer(nbytes=nbytes)) for _ in range(sets)]
    lib = eden.load()
    return dict(name="copy_%dMiB" % mib, launch=lambda s, i: eden.check(lib.eh_d2d(bufs[i][1].ptr, bufs[i][0].ptr, nbytes, s)),
                keep=bufs, sets=sets, ops=0.0, bytes=2 * nbytes, bound="hbm")


def stream_workload(eden, synth, mode=1, out_bytes=32 * 56 * 56 * 144, cold=False):
    """A kernel that only moves bytes in the ratio of an HBM-bound layer (mode 1: one chunk read, six written, the
    24 -> 144 pointwise layer; mode 2: four read, one written, the stride-2 depthwise layer; mode 0: copy): what the
    device gives a launch of that size before any arithmetic."""
    in_bytes = {0: out_bytes, 1: out_bytes // 6, 2: 4 * out_bytes}[mode]
    sets = set_count(in_bytes + out_bytes, cold)
    bufs = [(eden.DeviceBuffer(nbytes=in_bytes), eden.DeviceBuffer(nbytes=out_bytes)) for _ in range(sets)]
    for src, _ in bufs:
        eden.check(eden.load().eh_memset(src.ptr, 7, in_bytes, None))
    lib = eden.load()
    return dict(name="stream_%s_%.1fMB" % ({0: "copy", 1: "1to6", 2: "4to1"}[mode], (in_bytes + out_bytes) / 1e6),
                launch=lambda s, i: eden.check(lib.eh_probe_stream(bufs[i][0].ptr, bufs[i][1].ptr, out_bytes, mode, s)),
                keep=bufs, sets=sets, ops=0.0, bytes=in_bytes + out_bytes, bound="hbm")


def layout_workload(eden, synth, to_nhwc=True, n=64, c=96, h=112, w=112, cold=False):
    """NCHW <-> NHWC conversion of a feature map (MobileNetV2's largest, [64, 96, 112, 112]): bytes in + bytes out."""
    nbytes = n * c * h * w
    x = synth.fill_u8((nbytes,), SEED + 90)
    sets = set_count(2 * nbytes, cold)
    bufs = [(eden.DeviceBuffer(host=x), eden.DeviceBuffer(nbytes=nbytes)) for _ in range(sets)]
    lib = eden.load()
    fn = lib.eh_transpose_u8_nchw2nhwc if to_nhwc else lib.eh_transpose_u8_nhwc2nchw
    return dict(name="%s_n%d_c%d_%dx%d" % ("nchw2nhwc" if to_nhwc else "nhwc2nchw", n, c, h, w),
                launch=lambda s, i: eden.check(fn(bufs[i][0].ptr, bufs[i][1].ptr, n, c, h, w, s)),
                keep=bufs, sets=sets, ops=0.0, bytes=2 * nbytes, bound="hbm")


def roofline(work, event_s, steps):
    per_launch = event_s / steps
    if work["bound"] == "mfma":
        achieved = work["ops"] / per_launch / 1e12
        return dict(bound="mfma", achieved=round(achieved, 2), peak=INT8_PEAK_TOPS, unit="TOP/s",
                    frac=round(achieved / INT8_PEAK_TOPS, 4), us_per_launch=round(per_launch * 1e6, 3))
    achieved = work["bytes"] / per_launch / 1e9
    return dict(bound="hbm", achieved=round(achieved, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                frac=round(achieved / HBM_PEAK_GBS, 4), us_per_launch=round(per_launch * 1e6, 3))


def profiled_traffic():
    """HBM bytes per launch of the headline kernel, read from the committed rocprofv3 summary (FETCH_SIZE and
    WRITE_SIZE per dispatch, each scaled by what the same counter reads on a copy of known size); None without it."""
    try:
        text = open(HEADLINE_PROFILE).read()
        fetch = re.search(r"FETCH_SIZE.*= (\d+) bytes per dispatch", text)
        write = re.search(r"WRITE_SIZE.*= (\d+) bytes per dispatch", text)
        return int(fetch.group(1)) + int(write.group(1))
    except Exception:
        return None


def cpu_baseline(work):
    """The CPU oracle (a port of the reference semantics; the reference has no CPU kernels for
    this path) on the full headline GEMM, all host threads, median over about ten seconds of runs after one warm-up."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib as O
    a, w, b, q = work["host"]
    oq = O.Quant(*q.as_tuple())
    O.fc(a[:16], w, b, oq)
    times = []
    while sum(times) < 10.0 and len(times) < 2000:
        t0 = time.perf_counter()
        ref = O.fc(a, w, b, oq)
        times.append(time.perf_counter() - t0)
    got = work["out"].download(work["out_shape"])
    if not np.array_equal(got, ref):
        raise SystemExit("bench: GPU output differs from the CPU oracle")
    t = statistics.median(times)
    return dict(value=round(work["ops"] / t / 1e12, 4), unit="TOPS", cores=O.lib.eo_num_threads(), kind="port",
                sample="full workload (M=256, K=4096, N=4096) %d times, median %.4f s per run, %.1f s of CPU time in all; GPU output checked equal" % (len(times), t, sum(times)))


def check_network(work, userdriver=None):
    """The checker's part of the MobileNetV2 line: the network object that is about to be timed (batch 64) runs eight
    distinct images scattered over its batch positions (seeded, without a period) and the logits at every position
    must equal the CPU oracle's for the image that sits there; so must the logits of the same batch run through the
    userdriver's operator list when one is given.  The oracle's own time for the eight images is the CPU figure.
    Raises SystemExit on a mismatch."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from harness import oracle_forward, scattered_batch
    mobilenet = importlib.import_module("cl-eden-kernel_amd.mobilenet")
    net = work["net"]
    distinct = mobilenet.network_input(8)
    t0 = time.perf_counter()
    _, _, want = oracle_forward(distinct, 224, work["per_channel"], work["weights"])
    cpu_s = time.perf_counter() - t0
    where = scattered_batch(net.batch, 8)
    x = np.ascontiguousarray(distinct[where])
    ref = want[-1].reshape(8, -1)[where]
    net.set_input(x)
    net.run()
    eden_mod.sync(None)
    if not np.array_equal(net.logits(), ref):
        raise SystemExit("bench: %s: logits differ from the CPU oracle" % work["name"])
    net.set_input(mobilenet.network_input(net.batch))
    if userdriver is not None:
        driver, list_id, shape = userdriver
        driver.write_input(list_id, 0, x)
        driver.execute_operators(list_id, 3)   # direct, recorded, replayed: the replay's logits are the ones read
        driver.synchronize()
        if not np.array_equal(driver.read_output(list_id, 0, shape), ref):
            raise SystemExit("bench: %s through the operator API: logits differ from the CPU oracle" % work["name"])
        driver.write_input(list_id, 0, mobilenet.network_input(net.batch))
    return round(8 / cpu_s, 2)


def measure(eden, synth, stream, make, steps, warmup, use_graph, cold_too):
    """One workload, warm and (for the memory-bound ones, when asked) cold."""
    w = make(eden, synth)
    wall, ev, reps = time_steps(eden, stream, w["launch"], steps, warmup, use_graph, w.get("chunk", 50))
    entry = dict(workload=w["name"], steps=steps, tops=round(w["ops"] * steps / wall / 1e12, 2), roofline=roofline(w, ev, steps))
    entry["roofline"]["buffers"] = "warm: one buffer set replayed (%.1f MB, below the 256 MB Infinity Cache)" % (w["bytes"] / 1e6)
    if "images" in w:
        entry["images_per_s"] = round(w["images"] * steps / wall, 1)
        entry["roofline"]["buffers"] = "one step streams %.0f MB of feature maps (each written once and read by the next operators) through a pool of %.0f MB" % (w["working_set"] / 1e6, w["pool_bytes"] / 1e6)
    if reps > 1:
        entry["timed_region_repeats"] = reps
    del w
    if cold_too:
        c = make(eden, synth, cold=True)
        steps = round_steps(steps, c["sets"], c.get("chunk", 50))
        wall2, ev2, reps2 = time_steps(eden, stream, c["launch"], steps, warmup, use_graph, c.get("chunk", 50), c["sets"])
        warm = entry["roofline"]
        entry["roofline"] = roofline(c, ev2, steps)
        entry["steps_cold"] = steps
        entry["roofline"]["buffers"] = "cold: %d buffer sets in rotation (%.0f MB between two uses of a set)" % (c["sets"], c["sets"] * c["bytes"] / 1e6)
        entry["roofline_warm"] = warm
        entry["tops"] = round(c["ops"] * steps / wall2 / 1e12, 2)
        del c
    return entry


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--no-graph", action="store_true", help="launch every step from the host instead of replaying a HIP graph")
    ap.add_argument("--no-others", action="store_true", help="time the headline workload only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline and the oracle check of the network")
    ap.add_argument("--only", default=None, help="time one named workload family only: fc, fcbig, conv, conv64, dw, dwbig, pw, pwbig, deconv, mbv2 (two lanes, measured pairs fused), mbv2plain / mbv2lanes / mbv2fused (neither / lanes only / fusion only), mbv2ud (the same through the operator API), mbv2narrow, mbv2pc, mbv2udpc, mbv2b1 / mbv2b8 (the network at batch 1 and 8, one chain: latency), dwdil2, conv21, deconv21 (an atrous depthwise layer and a 21-class segmentation head), copy, tonhwc, tonchw, feedprobe (what a CU's matrix pipe can be fed with, per tile shape)")
    ap.add_argument("--tile", default=None, help="with --only c3block / block:...: ROWSxCOLS output pixels per workgroup (default: chosen by the library)")
    ap.add_argument("--cold", action="store_true", help="with --only: rotate over buffer sets that together exceed the Infinity Cache")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (got --gpus %d); no multi-GPU figure exists" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    global eden_mod
    eden = eden_mod = importlib.import_module("cl-eden-kernel_amd")
    synth = importlib.import_module("cl-eden-kernel_amd.synth")
    eden.init(0)
    stream = eden.Stream()
    use_graph = not args.no_graph

    def shaped(fn, **fixed):
        return lambda e, s, cold=False: fn(e, s, cold=cold, **fixed)

    families = dict(fc=fc_workload, conv=conv_workload, dw=dw_workload, pw=pw_workload, deconv=deconv_workload,
                    fcbig=shaped(fc_workload, m=8192, k=4096, n=4096), fc1=shaped(fc_workload, m=1, k=4096, n=4096), conv64=shaped(conv_workload, n=64),
                    c3block=block_workload, pw14=shaped(pw_workload, n=64, cin=64, cout=384, hw=14), pj14=shaped(pw_workload, n=64, cin=384, cout=64, hw=14),
                    pw7=shaped(pw_workload, n=64, cin=160, cout=960, hw=7), pj7=shaped(pw_workload, n=64, cin=960, cout=160, hw=7),
                    c3blockbig=shaped(block_workload, n=256),
                    dwbig=shaped(dw_workload, n=256), pwbig=shaped(pw_workload, n=256),
                    stem7x7=shaped(conv_workload, n=64, cin=3, cout=64, hw=224, k=7, stride=2),
                    dw5x5=shaped(dw_workload, n=64, c=144, hw=56, stride=1, k=5), dw7x7=shaped(dw_workload, n=64, c=144, hw=56, stride=1, k=7),
                    dwdil2=shaped(dw_workload, n=64, c=144, hw=56, stride=1, k=3, dil=2), conv21=shaped(conv_workload, n=8, cin=21, cout=21, hw=64, k=3, stride=1),
                    deconv21=shaped(deconv_workload, n=1, cin=21, cout=21, hw=64, k=16, stride=8),
                    copy=copy_workload, mbv2=mbv2_workload, mbv2narrow=shaped(mbv2_workload, weights="narrow"),
                    mbv2b1=shaped(mbv2_workload, batch=1, lanes=1), mbv2b8=shaped(mbv2_workload, batch=8, lanes=1),
                    tonhwc=layout_workload, tonchw=shaped(layout_workload, to_nhwc=False),
                    mbv2pc=shaped(mbv2_workload, per_channel=True),
                    mbv2plain=shaped(mbv2_workload, lanes=1, fuse_blocks=()), mbv2lanes=shaped(mbv2_workload, fuse_blocks=()),
                    mbv2fused=shaped(mbv2_workload, lanes=1),
                    stream16=stream_workload, stream16big=shaped(stream_workload, out_bytes=256 * 56 * 56 * 144),
                    stream41=shaped(stream_workload, mode=2, out_bytes=32 * 28 * 28 * 144),
                    stream41big=shaped(stream_workload, mode=2, out_bytes=256 * 28 * 28 * 144))
    if args.only == "feedprobe":
        # the yardsticks the GEMM tiles' inner loops are set against: one JSON line per mix
        for mix in range(len(eden.FEED_MIXES)):
            print(json.dumps(eden.probe_feed(mix, 256, 4000)), flush=True)
        return
    if args.only in ("mbv2ud", "mbv2udpc", "mbv2udplanar"):
        mobilenet = importlib.import_module("cl-eden-kernel_amd.mobilenet")
        driver, list_id, _ = mbv2_userdriver(eden, per_channel=args.only == "mbv2udpc", planar=args.only == "mbv2udplanar")
        if args.no_graph:
            driver.set_replay(False)
        steps = min(args.steps, 200)
        wall, ev, reps = time_userdriver(eden, driver, list_id, steps, max(3, min(args.warmup, 10)))
        print(json.dumps(dict(workload="mobilenet_v2_1.0_224_u8_batch64 through OperationConstructor / OperationExecutor", steps=steps,
                              ms_per_step=wall / steps * 1e3, us_per_step_by_events=ev / steps * 1e6, timed_region_repeats=reps,
                              images_per_s=round(64 * steps / wall, 1), executor=driver.stats(list_id))))
        return
    rows, cols = (int(v) for v in args.tile.split("x")) if args.tile else (0, 0)
    if args.only and args.tile:
        families["c3block"] = shaped(block_workload, rows=rows, cols=cols)
        families["c3blockbig"] = shaped(block_workload, n=256, rows=rows, cols=cols)
    if args.only and args.only.startswith("pw:"):      # pw:N,CIN,COUT,HW = that pointwise convolution
        n, cin, cout, hw = (int(v) for v in args.only[3:].split(","))
        families[args.only] = shaped(pw_workload, n=n, cin=cin, cout=cout, hw=hw)
    if args.only and args.only.startswith("fc:"):      # fc:M,K,N = that fully connected layer
        m, k, n = (int(v) for v in args.only[3:].split(","))
        families[args.only] = shaped(fc_workload, m=m, k=k, n=n)
    if args.only and args.only.startswith("deconv:"):  # deconv:N,CIN,COUT,HW,K,STRIDE = that transposed convolution
        n, cin, cout, hw, k, stride = (int(v) for v in args.only[7:].split(","))
        families[args.only] = shaped(deconv_workload, n=n, cin=cin, cout=cout, hw=hw, k=k, stride=stride)
    if args.only and args.only.startswith("conv:"):    # conv:N,CIN,COUT,HW,K,STRIDE[,DILATION] = that convolution
        v = [int(t) for t in args.only[5:].split(",")]
        families[args.only] = shaped(conv_workload, n=v[0], cin=v[1], cout=v[2], hw=v[3], k=v[4], stride=v[5], dil=v[6] if len(v) > 6 else 1)
    if args.only and args.only.startswith("dw:"):      # dw:N,C,HW,STRIDE[,K[,DILATION]] = that depthwise convolution
        v = [int(t) for t in args.only[3:].split(",")]
        families[args.only] = shaped(dw_workload, n=v[0], c=v[1], hw=v[2], stride=v[3], k=v[4] if len(v) > 4 else 3, dil=v[5] if len(v) > 5 else 1)
    if args.only and args.only.startswith(("block:", "twolaunch:")):
        # block:N,CIN,C,HW,STRIDE = that expansion + 3x3 depthwise pair as one launch; twolaunch: the same as two launches
        kind, _, spec = args.only.partition(":")
        n, cin, c, hw, stride = (int(v) for v in spec.split(","))
        families[args.only] = shaped(block_workload, n=n, cin=cin, c=c, hw=hw, stride=stride, rows=rows, cols=cols, fused=kind == "block")
    if args.only:
        work = families[args.only](eden, synth, cold=args.cold)
        args.steps = round_steps(args.steps, work["sets"], work.get("chunk", 50))
        wall, ev, reps = time_steps(eden, stream, work["launch"], args.steps, args.warmup, use_graph, work.get("chunk", 50), work["sets"])
        line = dict(workload=work["name"], steps=args.steps, ms_per_step=wall / args.steps * 1e3, buffer_sets=work["sets"],
                    timed_region_repeats=reps, roofline=roofline(work, ev, args.steps))
        if "images" in work:
            line["images_per_s"] = round(work["images"] * args.steps / wall, 1)
        print(json.dumps(line))
        return

    work = fc_workload(eden, synth)
    wall, ev, reps = time_steps(eden, stream, work["launch"], args.steps, args.warmup, use_graph)
    rf = roofline(work, ev, args.steps)
    rf["traffic"] = profiled_traffic()
    launch_note = "hip graph replay" if use_graph else "host launches"
    if reps > 1:
        launch_note += "; the %d steps took under %d ms, so the timed region is %d repetitions of them and ms_per_step is its wall clock / (%d x %d)" % (
            args.steps, int(MIN_TIMED_SECONDS * 1e3), reps, reps, args.steps)
    result = {
        "metric": "int8 TOPS per conv/FC layer + MobileNetV2-u8 images/sec, 1 GPU, % roofline",
        "value": round(work["ops"] * args.steps / wall / 1e12, 2),
        "unit": "TOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall / args.steps * 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8",
        "data": "synthetic",
        "config": {"workload": "uint8 FullyConnected GEMM M=256 K=4096 N=4096 (BASELINE configs[1]), int32 bias, "
                               "fixed-point requant fused, weights pre-packed, tensors resident in HBM",
                   "launch": launch_note},
        "roofline": rf,
    }
    # the ceilings measured on this device next to the published ones: int8 MFMA issued from registers only,
    # with constant operands and with operands whose bits toggle like data (sustained clocks differ)
    result["measured_peak"] = {"mfma_i8_constant_operands_tops": round(eden.probe_mfma_i8(200000, False), 1),
                               "mfma_i8_toggling_operands_tops": round(eden.probe_mfma_i8(200000, True), 1)}
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(work)
    del work
    if not args.no_others:
        # MobileNetV2 (BASELINE configs[4]): checked against the oracle before it is timed
        net = mbv2_workload(eden, synth)
        via_api = mbv2_userdriver(eden)
        if not args.no_cpu:
            result["cpu_baseline"]["mobilenet_v2_images_per_s"] = check_network(net, via_api)
            result["cpu_baseline"]["mobilenet_v2_sample"] = ("8 images (224x224x3) through the oracle's operator list; the batch-64 GPU network's logits checked equal, through "
                                                            "the C ABI and through the operator API, on those 8 images scattered over the 64 batch positions")
        wall2, ev2, reps2 = time_steps(eden, stream, net["launch"], 40, 4, use_graph, net["chunk"])
        c5 = dict(workload=net["name"], steps=40, tops=round(net["ops"] * 40 / wall2 / 1e12, 2), roofline=roofline(net, ev2, 40),
                  images_per_s=round(net["images"] * 40 / wall2, 1), checked_against_oracle=not args.no_cpu)
        c5["roofline"]["buffers"] = "one step streams %.0f MB of feature maps (each written once and read by the next operators) through a pool of %.0f MB" % (net["working_set"] / 1e6, net["pool_bytes"] / 1e6)
        c5["pool_bytes"] = net["pool_bytes"]
        c5["schedule"] = ("%d lanes of %d images on streams of their own, parallel branches of one graph; expansion + depthwise pairs run as one launch "
                          "(expanded tensor in LDS) at operators %s, chosen by eh_conv_dw_block_preferred" % (net["lanes"], net["images"] // net["lanes"], net["fused_blocks"]))
        # the same network built by OperationConstructor from an operator-list description and run by OperationExecutor
        if not use_graph:
            via_api[0].set_replay(False)
        wall3, ev3, reps3 = time_userdriver(eden, via_api[0], via_api[1], 40, 4)
        api_stats = via_api[0].stats(via_api[1])
        c5["operator_api"] = dict(path="eud_open_subgraph -> HipUserDriver -> OperationConstructor (HipComputeLibrary tensors and operators, pooled buffers) -> "
                                       "OperationExecutor (recorded once, replayed)", images_per_s=round(net["images"] * 40 / wall3, 1),
                                  us_per_batch_by_events=round(ev3 / 40 * 1e6, 1), executor=api_stats, checked_against_oracle=not args.no_cpu)
        result["images_per_s"] = c5["images_per_s"]
        result["images_per_s_operator_api"] = c5["operator_api"]["images_per_s"]
        result["config"]["images_per_s"] = c5["images_per_s"]
        result["config"]["images_per_s_operator_api"] = c5["operator_api"]["images_per_s"]
        result["config"]["images_per_s_workload"] = ("MobileNetV2-1.0 uint8 224x224x3, batch 64, per-tensor min/max quantized random-init weights "
                                                     "(BASELINE configs[4]); images_per_s: operator plans over the C ABI, one HIP graph replay per 4 batches, "
                                                     "ms per batch %.4f; images_per_s_operator_api: the operator list opened and executed through the "
                                                     "userdriver classes (OperationConstructor / OperationExecutor), ms per batch %.4f" % (wall2 / 40 * 1e3, wall3 / 40 * 1e3))
        via_api[0].close()
        del via_api
        # ... and as a planar list (feature maps [n, c, h, w], as Caffe-style models come): stored channels-last inside
        planar = mbv2_userdriver(eden, list_id=0xC6, planar=True)
        wall4, ev4, _ = time_userdriver(eden, planar[0], planar[1], 40, 4)
        c5["operator_api"]["planar_list"] = dict(images_per_s=round(net["images"] * 40 / wall4, 1), us_per_batch_by_events=round(ev4 / 40 * 1e6, 1),
                                                  executor=planar[0].stats(planar[1]))
        planar[0].close()
        del planar
        del net
        others = [c5]
        for make, steps, cold_too in ((conv_workload, 2000, False), (shaped(conv_workload, n=64), 300, False),
                                      (pw_workload, 500, True), (dw_workload, 1000, True), (block_workload, 500, True),
                                      (shaped(pw_workload, n=256), 100, True), (shaped(dw_workload, n=256), 200, True),
                                      (shaped(conv_workload, n=64, cin=3, cout=64, hw=224, k=7, stride=2), 200, False),
                                      (shaped(dw_workload, n=64, c=144, hw=56, stride=1, k=5), 200, False),
                                      (shaped(dw_workload, n=64, c=144, hw=56, stride=1, k=7), 200, False),
                                      # an atrous depthwise layer, and the shapes of a 21-class segmentation head (channel counts
                                      # that are no multiple of 16; an upsampling whose kernel is twice its stride)
                                      (shaped(dw_workload, n=64, c=144, hw=56, stride=1, k=3, dil=2), 200, False),
                                      (shaped(conv_workload, n=8, cin=21, cout=21, hw=64, k=3, stride=1), 500, False),
                                      (shaped(deconv_workload, n=1, cin=21, cout=21, hw=64, k=16, stride=8), 200, False),
                                      (deconv_workload, 500, False), (fc_workload, 500, True),
                                      (shaped(fc_workload, m=8192, k=4096, n=4096), 100, False),
                                      (shaped(fc_workload, m=1, k=4096, n=4096), 500, True),
                                      (layout_workload, 200, True), (shaped(layout_workload, to_nhwc=False), 200, True),
                                      (copy_workload, 200, True),
                                      (stream_workload, 500, True), (shaped(stream_workload, out_bytes=256 * 56 * 56 * 144), 100, True),
                                      (shaped(stream_workload, mode=2, out_bytes=32 * 28 * 28 * 144), 500, True),
                                      (shaped(stream_workload, mode=2, out_bytes=256 * 28 * 28 * 144), 100, True),
                                      # the network's latency: one image, and eight, as one chain
                                      (shaped(mbv2_workload, batch=1, lanes=1), 200, False), (shaped(mbv2_workload, batch=8, lanes=1), 200, False),
                                      (shaped(mbv2_workload, weights="narrow"), 40, False),
                                      (shaped(mbv2_workload, per_channel=True), 40, False)):
            others.append(measure(eden, synth, stream, make, steps, max(4, steps // 10), use_graph, cold_too))
        result["others"] = others
        # the headline workload on cold buffers (sets rotated so that nothing is found in the Infinity Cache), beside the
        # warm figure `value` and `roofline` are measured on
        for entry in others:
            if entry["workload"] == "fc_m256_k4096_n4096" and "roofline_warm" in entry:
                result["roofline_cold"] = entry["roofline"]
    result["roofline"]["buffers"] = "warm: one set of tensors replayed; the 16 MiB of weights are found in the 256 MB Infinity Cache (roofline_cold: rotated sets)"
    print(json.dumps(result))


if __name__ == "__main__":
    main()
