"""Benchmark of the quantized operator hot path on one MI355X.

Headline workload (BASELINE.json configs[1]): uint8 FullyConnected GEMM, M=256
batch rows, K=4096, N=4096, zero points 3 / 128, scales 0.01 / 0.002 / 0.08,
int32 bias, fixed-point requantization fused.  One step = one execution of the
operator on device-resident tensors with pre-packed weights.  The other
configurations are timed the same way and reported under "others".

Prints ONE JSON line.  `--gpus N` with N > 1 is refused: this build uses one GPU."""
import argparse
import importlib
import json
import os
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

INT8_PEAK_TOPS = 5000.0   # MI355X dense int8 MFMA peak, TOP/s
HBM_PEAK_GBS = 8000.0     # MI355X HBM3E peak, GB/s
SEED = 0xEDE2
# HBM bytes per launch of the headline kernel from rocprofv3 --pmc (FETCH_SIZE 12348.6 KiB x 1.999,
# WRITE_SIZE 1024 KiB x 1.000, the factors being what the same counters read on a 64 MiB copy):
# profiles/igemm_dma_64x64_splitk__fc_m256_k4096_n4096.md
MEASURED_TRAFFIC_BYTES = 25281004 + 1048576


def time_steps(eden, stream, launch, steps, warmup, use_graph=True, chunk=50):
    """Runs `warmup` untimed and exactly `steps` timed executions of launch(stream_handle).
    Returns (wall seconds, HIP-event seconds) for the timed region."""
    for _ in range(warmup):
        launch(stream.h)
    stream.sync()
    graph = None
    chunk = max(1, min(chunk, steps))
    if use_graph:
        graph = eden.Graph(stream, lambda s: [launch(s) for _ in range(chunk)])
        graph.launch(stream)  # first replay uploads the graph; keep it out of the timed region
        stream.sync()
    e0, e1 = eden.Event(), eden.Event()
    device_sync()
    t0 = time.perf_counter()
    e0.record(stream.h)
    done = 0
    if graph is not None:
        while done + chunk <= steps:
            graph.launch(stream)
            done += chunk
    while done < steps:
        launch(stream.h)
        done += 1
    e1.record(stream.h)
    stream.sync()
    device_sync()
    t1 = time.perf_counter()
    return t1 - t0, e1.elapsed_ms_since(e0) * 1e-3


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


def fc_workload(eden, synth, m=256, k=4096, n=4096):
    a = synth.fill_u8((m, k), SEED + 32)
    w = synth.fill_u8_normal((n, k), SEED + 33, 128, 20)
    b = synth.fill_i32((n,), SEED + 34, -1000, 1000)
    q = eden.make_requant(0.01, 3, 0.002, 128, 0.08, 0)
    d_a, d_w, d_b = eden.DeviceBuffer(host=a), eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
    d_o = eden.DeviceBuffer(nbytes=m * n)
    plan = eden.FcPlan(m, k, n, d_w, d_b, q)
    keep = (d_a, d_w, d_b, d_o, plan)
    return dict(name="fc_m%d_k%d_n%d" % (m, k, n), launch=lambda s: plan.run(d_a, d_o, q, s), keep=keep,
                ops=2.0 * m * k * n, bytes=m * k + n * k + 4 * n + m * n, bound="mfma",
                host=(a, w, b, q), out=d_o, out_shape=(m, n))


def conv_workload(eden, synth, n=1):
    desc = eden.conv_desc(n, 64, 56, 56, 64, 3, 3, pad=(1, 1, 1, 1), layout=eden.NHWC)
    x = synth.fill_u8((n, 56, 56, 64), SEED + 16)
    w = synth.fill_u8((64, 64, 3, 3), SEED + 17)
    b = synth.fill_i32((64,), SEED + 18, -1000, 1000)
    q = eden.make_requant(0.02, 128, 0.005, 120, 0.05, 0, eden.ACT_RELU, True)
    d_x, d_w, d_b = eden.DeviceBuffer(host=x), eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
    d_o = eden.DeviceBuffer(nbytes=n * 56 * 56 * 64)
    plan = eden.ConvPlan(desc, d_w, d_b, q)
    return dict(name="conv3x3_n%d_c64_56x56_nhwc" % n, launch=lambda s: plan.run(d_x, d_o, q, s),
                keep=(d_x, d_w, d_b, d_o, plan), ops=2.0 * n * 56 * 56 * 64 * 576,
                bytes=2 * n * 56 * 56 * 64 + 64 * 576 + 256, bound="mfma")


def dw_workload(eden, synth, n=32):
    desc = eden.conv_desc(n, 144, 56, 56, 144, 3, 3, stride=(2, 2), pad=(1, 1, 1, 1), dm=1, layout=eden.NHWC)
    x = synth.fill_u8((n, 56, 56, 144), SEED + 48)
    w = synth.fill_u8((144, 1, 3, 3), SEED + 49)
    b = synth.fill_i32((144,), SEED + 50, -1000, 1000)
    q = eden.make_requant(0.03, 17, 0.006, 140, 0.025, 9, eden.ACT_RELU6, True)
    d_x, d_w, d_b = eden.DeviceBuffer(host=x), eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
    d_o = eden.DeviceBuffer(nbytes=n * 28 * 28 * 144)
    plan = eden.DwConvPlan(desc, d_w, d_b, q)
    return dict(name="dw3x3s2_n%d_c144_56x56_nhwc" % n, launch=lambda s: plan.run(d_x, d_o, q, s),
                keep=(d_x, d_w, d_b, d_o, plan), ops=2.0 * n * 144 * 28 * 28 * 9,
                bytes=n * 144 * 56 * 56 + 144 * 9 + 144 * 4 + n * 144 * 28 * 28, bound="hbm")


def pw_workload(eden, synth, n=32):
    desc = eden.conv_desc(n, 24, 56, 56, 144, 1, 1, layout=eden.NHWC)
    x = synth.fill_u8((n, 56, 56, 24), SEED + 51)
    w = synth.fill_u8((144, 24, 1, 1), SEED + 52)
    b = synth.fill_i32((144,), SEED + 53, -1000, 1000)
    q = eden.make_requant(0.02, 120, 0.004, 131, 0.03, 4, eden.ACT_RELU6, True)
    d_x, d_w, d_b = eden.DeviceBuffer(host=x), eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
    d_o = eden.DeviceBuffer(nbytes=n * 56 * 56 * 144)
    plan = eden.ConvPlan(desc, d_w, d_b, q)
    return dict(name="pw1x1_n%d_24to144_56x56_nhwc" % n, launch=lambda s: plan.run(d_x, d_o, q, s),
                keep=(d_x, d_w, d_b, d_o, plan), ops=2.0 * n * 56 * 56 * 24 * 144,
                bytes=n * 56 * 56 * 24 + 144 * 24 + 576 + n * 56 * 56 * 144, bound="hbm")


def deconv_workload(eden, synth, n=8):
    desc = eden.conv_desc(n, 256, 32, 32, 128, 4, 4, stride=(2, 2), pad=(1, 1, 1, 1), layout=eden.NHWC,
                          weight_layout=eden.W_IOHW)
    x = synth.fill_u8((n, 32, 32, 256), SEED + 64)
    w = synth.fill_u8((256, 128, 4, 4), SEED + 65)
    b = synth.fill_i32((128,), SEED + 66, -1000, 1000)
    q = eden.make_requant(0.02, 121, 0.005, 133, 0.35, 128)
    d_x, d_w, d_b = eden.DeviceBuffer(host=x), eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
    d_o = eden.DeviceBuffer(nbytes=n * 64 * 64 * 128)
    plan = eden.DeconvPlan(desc, d_w, d_b, q)
    return dict(name="deconv4x4s2_n%d_256to128_32x32_nhwc" % n, launch=lambda s: plan.run(d_x, d_o, q, s),
                keep=(d_x, d_w, d_b, d_o, plan), ops=2.0 * n * 1024 * 256 * 2048,
                bytes=n * 256 * 1024 + 256 * 128 * 16 + 512 + n * 128 * 4096, bound="mfma")


def mbv2_workload(eden, synth, batch=64, per_channel=False):
    """BASELINE.json configs[4]: MobileNetV2-1.0 uint8 at 224x224x3, batch 64, the whole operator list per step.
    per_channel: int8 weights with one scale per output channel in the convolutions."""
    mobilenet = importlib.import_module("cl-eden-kernel_amd.mobilenet")
    # residual adds inside the projection convolutions' launches
    net = mobilenet.MobileNetV2(eden, batch, fuse_add=True, per_channel=per_channel)
    net.set_input(mobilenet.network_input(batch))
    return dict(name="mobilenet_v2_1.0_224_u8%s_batch%d" % ("_perchannel_w" if per_channel else "", batch), launch=lambda s: net.run(s), keep=net,
                ops=2.0 * mobilenet.macs_per_image() * batch, bytes=mobilenet.compulsory_bytes_per_image() * batch,
                bound="hbm", images=batch, chunk=4)


def copy_workload(eden, synth, mib=64):
    """A plain device-to-device copy of known size: the yardstick the HBM byte counters are scaled by."""
    nbytes = mib << 20
    src, dst = eden.DeviceBuffer(nbytes=nbytes), eden.DeviceBuffer(nbytes=nbytes)
    lib = eden.load()
    return dict(name="copy_%dMiB" % mib, launch=lambda s: eden.check(lib.eh_d2d(dst.ptr, src.ptr, nbytes, s)),
                keep=(src, dst), ops=0.0, bytes=2 * nbytes, bound="hbm")


def layout_workload(eden, synth, to_nhwc=True, n=64, c=96, h=112, w=112):
    """NCHW <-> NHWC conversion of a feature map (MobileNetV2's largest, [64, 96, 112, 112]): bytes in + bytes out."""
    nbytes = n * c * h * w
    src, dst = eden.DeviceBuffer(host=synth.fill_u8((nbytes,), SEED + 90)), eden.DeviceBuffer(nbytes=nbytes)
    lib = eden.load()
    fn = lib.eh_transpose_u8_nchw2nhwc if to_nhwc else lib.eh_transpose_u8_nhwc2nchw
    return dict(name="%s_n%d_c%d_%dx%d" % ("nchw2nhwc" if to_nhwc else "nhwc2nchw", n, c, h, w),
                launch=lambda s: eden.check(fn(src.ptr, dst.ptr, n, c, h, w, s)),
                keep=(src, dst), ops=0.0, bytes=2 * nbytes, bound="hbm")


def roofline(work, event_s, steps):
    per_launch = event_s / steps
    if work["bound"] == "mfma":
        achieved = work["ops"] / per_launch / 1e12
        return dict(bound="mfma", achieved=round(achieved, 2), peak=INT8_PEAK_TOPS, unit="TOP/s",
                    frac=round(achieved / INT8_PEAK_TOPS, 4), us_per_launch=round(per_launch * 1e6, 3))
    achieved = work["bytes"] / per_launch / 1e9
    return dict(bound="hbm", achieved=round(achieved, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                frac=round(achieved / HBM_PEAK_GBS, 4), us_per_launch=round(per_launch * 1e6, 3))


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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--no-graph", action="store_true", help="launch every step from the host instead of replaying a HIP graph")
    ap.add_argument("--no-others", action="store_true", help="time the headline workload only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--only", default=None, help="time one named workload family only: fc, fcbig, conv, conv64, dw, pw, deconv, mbv2, mbv2pc, copy, tonhwc, tonchw")
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

    families = dict(fc=fc_workload, conv=conv_workload, dw=dw_workload, pw=pw_workload, deconv=deconv_workload,
                    fcbig=lambda e, s: fc_workload(e, s, 8192, 4096, 4096), conv64=lambda e, s: conv_workload(e, s, 64),
                    copy=copy_workload, mbv2=mbv2_workload, tonhwc=layout_workload,
                    tonchw=lambda e, s: layout_workload(e, s, to_nhwc=False),
                    mbv2pc=lambda e, s: mbv2_workload(e, s, per_channel=True))
    if args.only:
        work = families[args.only](eden, synth)
        wall, ev = time_steps(eden, stream, work["launch"], args.steps, args.warmup, use_graph, work.get("chunk", 50))
        line = dict(workload=work["name"], steps=args.steps, ms_per_step=wall / args.steps * 1e3,
                    roofline=roofline(work, ev, args.steps))
        if "images" in work:
            line["images_per_s"] = round(work["images"] * args.steps / wall, 1)
        print(json.dumps(line))
        return

    work = fc_workload(eden, synth)
    wall, ev = time_steps(eden, stream, work["launch"], args.steps, args.warmup, use_graph)
    rf = roofline(work, ev, args.steps)
    rf["traffic"] = MEASURED_TRAFFIC_BYTES
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
                   "launch": "hip graph replay" if use_graph else "host launches"},
        "roofline": rf,
    }
    # the ceilings measured on this device next to the published ones: int8 MFMA issued from registers only,
    # with constant operands and with operands whose bits toggle like data (sustained clocks differ)
    result["measured_peak"] = {"mfma_i8_constant_operands_tops": round(eden.probe_mfma_i8(200000, False), 1),
                               "mfma_i8_toggling_operands_tops": round(eden.probe_mfma_i8(200000, True), 1)}
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(work)
    if not args.no_others:
        others = []
        for make, steps in ((conv_workload, 2000), (lambda e, s: conv_workload(e, s, 64), 300), (pw_workload, 500),
                            (dw_workload, 1000), (deconv_workload, 500),
                            (lambda e, s: fc_workload(e, s, 8192, 4096, 4096), 100),
                            (layout_workload, 200), (lambda e, s: layout_workload(e, s, to_nhwc=False), 200),
                            (mbv2_workload, 40),
                            (lambda e, s: mbv2_workload(e, s, per_channel=True), 40)):
            w2 = make(eden, synth)
            wall2, ev2 = time_steps(eden, stream, w2["launch"], steps, max(10, steps // 10), use_graph, w2.get("chunk", 50))
            entry = dict(workload=w2["name"], steps=steps, tops=round(w2["ops"] * steps / wall2 / 1e12, 2),
                         roofline=roofline(w2, ev2, steps))
            if "images" in w2:
                entry["images_per_s"] = round(w2["images"] * steps / wall2, 1)
            others.append(entry)
            del w2
        result["others"] = others
    print(json.dumps(result))


if __name__ == "__main__":
    main()
