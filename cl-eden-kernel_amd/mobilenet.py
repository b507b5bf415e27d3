"""MobileNetV2-1.0 (224x224x3, 1000 classes) as a list of quantized uint8
operators over the C ABI: convolution, depthwise convolution, pointwise
convolution, residual Add, AveragePool and FullyConnected, per-tensor
asymmetric quantization, ReLU6 as a clamp in the quantized domain.

The operator list plays the part of the reference's OperationConstructor /
OperationExecutor pair (src/userdriver/gpu/gpu_op_constructor.cc:1797-1850,
gpu_userdriver.cc:78-112): build every operator once, then execute them in
order on one stream, here captured into one HIP graph.

Weights are random (there is no checkpoint).  The default form ("minmax") is
what a post-training quantizer makes of random-init float weights: a zero-mean
normal field per tensor, its minimum mapped to byte 0 and its maximum to byte
255, the zero point where real 0 falls, so the bytes of every tensor span
0 .. 255.  The "narrow" form (uint8 clip(round(N(zp_w, 20))) with a per-layer
zero point, every byte within int8 reach of its zero point) is kept as a
labelled extra.  Bias is int32 uniform.  Scales are chosen analytically from the layer shapes so that activations neither die nor saturate
on their way through the 53 convolutions:
  * a ReLU6 output tensor has zero point 0 and scale 6/255, so ReLU6 is the
    whole uint8 range, and the layer's weight scale is set so that the
    pre-activation has a standard deviation of about 64 output steps;
  * a linear (projection / classifier) output has zero point 128 and about 30
    steps of standard deviation;
  * a residual sum is rescaled back to about 30 steps.
`layers()` is pure data (no GPU): tests evaluate the same list with the oracle.
"""
import functools
import math

import numpy as np

from . import synth

SEED = 0xEDE2 + 16 * 5

# (expansion t, output channels c, repeats n, stride s)
BOTTLENECKS = ((1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2), (6, 320, 1, 1))

W_SD = 20                 # "narrow" weights: standard deviation of the weight bytes around their zero point
FIELD_SD = 65535          # standard deviation of the integer normal field the "minmax" weights are quantized from
RELU6_SCALE = 6.0 / 255   # ReLU6 == [0, 255] at zero point 0
RELU_RMS = 45.0           # root mean square of clip(N(0, 64), 0, 255)
LINEAR_SD = 30.0
INPUT_SCALE, INPUT_ZP = 0.02, 128
INPUT_RMS = 74.0          # of uniform bytes around 128


@functools.lru_cache(maxsize=None)
def _field_extremes(shape, seed):
    g = synth.fill_normal_field(shape, seed)
    return int(g.min()), int(g.max())


def _minmax_bytes(g, lo, hi):
    """round((g - lo) * 255 / (hi - lo)) in integer arithmetic"""
    span = hi - lo
    return ((2 * 255 * (g - lo) + span) // (2 * span)).astype(np.uint8)


def layers(image=224, weights="minmax"):
    """The operator list.  Tensors are numbered; tensor 0 is the network input.  Returns
    (tensors, ops): tensors[i] = dict(h, w, c, scale, zp, rms), ops = list of dicts.
    weights: "minmax" (per-tensor min/max quantized, bytes span 0 .. 255) or "narrow"."""
    assert weights in ("minmax", "narrow")
    tensors = [dict(h=image, w=image, c=3, scale=INPUT_SCALE, zp=INPUT_ZP, rms=INPUT_RMS)]
    ops = []

    def weight_stats(shape, seed, narrow_zp):
        """(zero point, standard deviation of the bytes around it) of an operator's weight tensor"""
        if weights == "narrow":
            return narrow_zp, float(W_SD)
        lo, hi = _field_extremes(shape, seed)
        return int((2 * 255 * (0 - lo) + (hi - lo)) // (2 * (hi - lo))), FIELD_SD * 255.0 / (hi - lo)

    def conv(src, cout, k, stride, relu6, depthwise=False):
        t = tensors[src]
        idx = len(ops)
        pad = (k - 1) // 2
        ho, wo = (t["h"] + 2 * pad - k) // stride + 1, (t["w"] + 2 * pad - k) // stride + 1
        fan_in = k * k * (1 if depthwise else t["c"])
        w_seed = SEED + 3 * idx
        w_zp, w_sd = weight_stats((cout, 1 if depthwise else t["c"], k, k), w_seed, 120 + idx % 16)
        acc_sd = math.sqrt(fan_in) * w_sd * t["rms"]
        if relu6:
            out_scale, out_zp, out_sd, out_rms = RELU6_SCALE, 0, 64.0, RELU_RMS
        else:
            out_scale, out_zp, out_sd, out_rms = 0.05, 128, LINEAR_SD, LINEAR_SD
        w_scale = (out_sd / acc_sd) * out_scale / t["scale"]
        tensors.append(dict(h=ho, w=wo, c=cout, scale=out_scale, zp=out_zp, rms=out_rms))
        ops.append(dict(op="dw" if depthwise else "conv", src=src, dst=len(tensors) - 1, k=k, stride=stride, pad=pad,
                        cout=cout, relu6=relu6, w_scale=w_scale, w_zp=w_zp, w_seed=w_seed, w_mode=weights,
                        b_seed=SEED + 3 * idx + 1, b_range=max(1, int(acc_sd / 4))))
        return len(tensors) - 1

    cur = conv(0, 32, 3, 2, True)
    for t_exp, c, n, s in BOTTLENECKS:
        for rep in range(n):
            block_in = cur
            cin = tensors[cur]["c"]
            x = cur
            if t_exp != 1:
                x = conv(x, cin * t_exp, 1, 1, True)
            x = conv(x, tensors[x]["c"], 3, s if rep == 0 else 1, True, depthwise=True)
            x = conv(x, c, 1, 1, False)
            if rep > 0 and cin == c:   # stride 1 and equal shapes: residual connection
                a, b = tensors[block_in], tensors[x]
                real_sd = math.hypot(a["rms"] * a["scale"], b["rms"] * b["scale"])
                tensors.append(dict(h=b["h"], w=b["w"], c=c, scale=real_sd / LINEAR_SD, zp=128, rms=LINEAR_SD))
                ops.append(dict(op="add", a=block_in, b=x, dst=len(tensors) - 1))
                x = len(tensors) - 1
            cur = x
    cur = conv(cur, 1280, 1, 1, True)
    t = tensors[cur]
    tensors.append(dict(h=1, w=1, c=t["c"], scale=t["scale"], zp=t["zp"], rms=30.0))
    ops.append(dict(op="avgpool", src=cur, dst=len(tensors) - 1, k=t["h"]))
    cur = len(tensors) - 1
    t = tensors[cur]
    idx = len(ops)
    w_zp, w_sd = weight_stats((1000, t["c"]), SEED + 3 * idx, 128)
    acc_sd = math.sqrt(t["c"]) * w_sd * t["rms"]
    tensors.append(dict(h=1, w=1, c=1000, scale=0.05, zp=128, rms=LINEAR_SD))
    ops.append(dict(op="fc", src=cur, dst=len(tensors) - 1, cout=1000, w_scale=(LINEAR_SD / acc_sd) * 0.05 / t["scale"],
                    w_zp=w_zp, w_seed=SEED + 3 * idx, w_mode=weights, b_seed=SEED + 3 * idx + 1, b_range=max(1, int(acc_sd / 4))))
    return tensors, ops


def op_weights(op, cin):
    """(weights, bias) of a conv / dw / fc operator: OIHW uint8 (depthwise: [C, 1, k, k]; fc: [N, K]) and int32."""
    if op["op"] == "fc":
        shape = (op["cout"], cin)
    elif op["op"] == "dw":
        shape = (op["cout"], 1, op["k"], op["k"])
    else:
        shape = (op["cout"], cin, op["k"], op["k"])
    if op["w_mode"] == "minmax":
        w = _minmax_bytes(synth.fill_normal_field(shape, op["w_seed"]), *_field_extremes(shape, op["w_seed"]))
    else:
        w = synth.fill_u8_normal(shape, op["w_seed"], op["w_zp"], W_SD)
    b = synth.fill_i32((op["cout"],), op["b_seed"], -op["b_range"], op["b_range"])
    return w, b


def op_weights_perchannel(op, cin):
    """(int8 weights, bias, float32 scale per output channel) of a conv / dw operator in the per-channel form
    (int8 weights at zero point 0, as TFLite's full-integer converter writes them).  "minmax": the operator's normal
    field with every channel's largest magnitude mapped to 127 (bytes span -127 .. 127 in every channel), the
    channel's scale following from it.  "narrow": clip(round(N(0, 20))) and the layer's weight scale times a factor
    in [0.5, 2] per channel."""
    shape = (op["cout"], 1 if op["op"] == "dw" else cin, op["k"], op["k"])
    b = synth.fill_i32((op["cout"],), op["b_seed"], -op["b_range"], op["b_range"])
    if op["w_mode"] == "minmax":
        g = synth.fill_normal_field(shape, op["w_seed"]).reshape(op["cout"], -1)
        top = np.maximum(np.abs(g).max(axis=1, keepdims=True), 1)
        num = 2 * 127 * np.abs(g) + top
        w = (np.sign(g) * (num // (2 * top))).astype(np.int8).reshape(shape)
        lo, hi = _field_extremes(shape, op["w_seed"])
        field_step = op["w_scale"] * 255.0 / (hi - lo)   # real value of one unit of the field
        return w, b, (top.reshape(-1).astype(np.float64) * field_step / 127.0).astype(np.float32)
    w = (synth.fill_u8_normal(shape, op["w_seed"], 128, W_SD).astype(np.int16) - 128).clip(-127, 127).astype(np.int8)
    factor = 0.5 + 1.5 * synth.fill_u8((op["cout"],), op["w_seed"] + 2).astype(np.float32) / 255.0
    return w, b, (np.float32(op["w_scale"]) * factor).astype(np.float32)


def network_input(batch, image=224):
    """uint8 uniform[0, 255], channels-last [batch, image, image, 3]"""
    return synth.fill_u8((batch, image, image, 3), SEED + 9999)


def macs_per_image(image=224):
    tensors, ops = layers(image)
    total = 0
    for op in ops:
        if op["op"] in ("conv", "dw", "fc"):
            d = tensors[op["dst"]]
            cin = tensors[op["src"]]["c"]
            k2 = op.get("k", 1) ** 2
            total += d["h"] * d["w"] * d["c"] * k2 * (1 if op["op"] == "dw" else cin)
    return total


def compulsory_bytes_per_image(image=224):
    """activations in and out of every operator, once each (weights excluded: they are shared by the batch)"""
    tensors, ops = layers(image)
    size = lambda i: tensors[i]["h"] * tensors[i]["w"] * tensors[i]["c"]
    total = 0
    for op in ops:
        srcs = [op["a"], op["b"]] if op["op"] == "add" else [op["src"]]
        total += sum(size(i) for i in srcs) + size(op["dst"])
    return total


def operator_list(ud, list_id, batch, image=224, per_channel=False, weights="minmax", nchw=False):
    """The same network as a description for the userdriver (`ud` = the userdriver module): an androidNN model with
    channels-last data (use_nchw false), i.e. feature maps [batch, h, w, c], convolution filters [out, kh, kw, in] and
    depthwise filters [1, kh, kw, c] as TFLite stores them, and the explicit padding values of layers() (its
    symmetric padding is not what SAME gives a stride-2 layer).  nchw: the same model with planar data (use_nchw true:
    feature maps [batch, c, h, w]; the filters stay as they are).  Returns (OperatorList, input buffer index, output
    buffer index, logits shape).  Buffer index i is tensor i of layers()."""
    tensors, ops = layers(image, weights)
    ol = ud.OperatorList(list_id, ud.MODEL_ANDROID_NN)
    fm = {}

    def feature_map(i):
        if i not in fm:
            t = tensors[i]
            shape = (batch, t["c"], t["h"], t["w"]) if nchw else (batch, t["h"], t["w"], t["c"])
            fm[i] = ol.feature_map(i, shape, t["scale"], t["zp"])
        return fm[i]

    for n, op in enumerate(ops):
        kind = op["op"]
        if kind == "add":
            ol.operator("ADD_%d" % n, ud.OP_ADD, [feature_map(op["a"]), feature_map(op["b"])], [feature_map(op["dst"])])
            continue
        s = tensors[op["src"]]
        if kind == "avgpool":
            ol.operator("AVERAGE_POOL_2D_%d" % n, ud.OP_AVERAGE_POOL_2D, [feature_map(op["src"])], [feature_map(op["dst"])],
                        ud.options(padding=ud.PADDING_VALID, stride=(1, 1), filter=(op["k"], op["k"]), use_nchw=nchw))
            continue
        act = ud.ACT_RELU6 if op.get("relu6") else ud.ACT_NONE
        bias_scale = float(np.float32(s["scale"]) * np.float32(op["w_scale"]))
        if kind == "fc":
            w, b = op_weights(op, s["c"])
            wt = ol.parameter(w, op["w_scale"], op["w_zp"])
            bt = ol.parameter(b, bias_scale, 0)
            ol.operator("FULLY_CONNECTED_%d" % n, ud.OP_FULLY_CONNECTED, [feature_map(op["src"]), wt, bt], [feature_map(op["dst"])],
                        ud.options(activation=act))
            continue
        if per_channel:
            w, b, w_scales = op_weights_perchannel(op, s["c"])
        else:
            (w, b), w_scales = op_weights(op, s["c"]), None
        if kind == "dw":
            w = np.ascontiguousarray(w.transpose(1, 2, 3, 0))   # [C, 1, kh, kw] -> [1, kh, kw, C]
        else:
            w = np.ascontiguousarray(w.transpose(0, 2, 3, 1))   # [O, I, kh, kw] -> [O, kh, kw, I]
        wt = ol.parameter(w, 0.0 if per_channel else op["w_scale"], 0 if per_channel else op["w_zp"], per_channel_scales=w_scales)
        bt = ol.parameter(b, 1.0 if per_channel else bias_scale, 0)
        pad = op["pad"]
        opts = ud.options(padding=ud.PADDING_VALID, stride=(op["stride"],) * 2, activation=act, padding_value=(pad,) * 4, use_nchw=nchw)
        code, name = (ud.OP_DEPTHWISE_CONV_2D, "DEPTHWISE_CONV_2D_%d") if kind == "dw" else (ud.OP_CONV_2D, "CONV_2D_%d")
        ol.operator(name % n, code, [feature_map(op["src"]), wt, bt], [feature_map(op["dst"])], opts)
    last = len(tensors) - 1
    return ol, 0, last, (batch, tensors[last]["c"])


class MobileNetV2:
    """The operator list instantiated on the GPU for one batch size.  Activations are channels-last.

    fuse_add: a residual Add whose second operand is the projection convolution right before it (and nothing else
    reads that projection) runs inside that convolution's launch (`ConvPlan.run_add`); the projection's own tensor
    is then never written.  Results are the same bit for bit.

    per_channel: convolutions and depthwise convolutions take int8 weights with one scale per output channel
    (`op_weights_perchannel`); tensors stay uint8 and the classifier keeps its per-tensor uint8 weights.

    pooled: feature maps live in the library's buffer pool as the reference's operator constructor places them
    (gpu_op_constructor.cc:2157-2191): an operator's output is requested with INTER_SHARED_REUSE, then the inputs it
    is the last reader of are handed back, and once the list is built one device allocation holds them all
    (`pool_bytes`).  A feature map's storage is then taken over by later ones (the network input is kept), so only
    the input and the logits can be read back after a run; without it every tensor keeps a buffer of its own (`tensor()` works for all).

    lanes, lane_from, lane_to: operators lane_from .. lane_to - 1 (default: all) run as `lanes` independent chains, each
    on its own share of the images (the batch is the outermost dimension, so a share is a contiguous slice of every
    tensor), with its own feature maps, and on its own stream, forked from the caller's stream and joined to it again.
    A launch ends in a tail during which most CUs idle and the next one takes a while to fill them; two chains fill
    those gaps for one another (measured at batch 64: 490 -> 444 us per step with two lanes over the whole list, four
    lanes of 16 images lose more in the smaller launches than they gain).  Captured in a
    graph the chains become parallel branches.  Same plans, same kernels, same results."""

    def __init__(self, eden, batch, image=224, stream=None, fuse_add=False, per_channel=False, weights="minmax", pooled=False,
                 lanes=1, lane_from=None, lane_to=None, fuse_blocks=()):
        self.eden, self.batch, self.image = eden, batch, image
        self.tensors, self.ops = layers(image, weights)
        self.steps = []
        self._keep = []
        self.unwritten = set()  # tensors a fused step skips
        self.pooled = pooled
        readers = {}
        for op in self.ops:
            for key in ("src", "a", "b"):
                if key in op:
                    readers[op[key]] = readers.get(op[key], 0) + 1
        # a fused convolution + add never stores the projection's own tensor: find those before placing buffers
        if fuse_add:
            for index, op in enumerate(self.ops):
                if (op["op"] == "add" and index > 0 and self.ops[index - 1]["op"] == "conv" and self.ops[index - 1]["dst"] == op["b"]
                        and readers.get(op["b"], 0) == 1):
                    self.unwritten.add(op["b"])
        lane_to = len(self.ops) if lane_to is None else lane_to
        lane_from = lane_to if lanes <= 1 else (0 if lane_from is None else lane_from)
        lanes = lanes if lane_from < lane_to else 1
        assert batch % lanes == 0 and 0 <= lane_from <= lane_to <= len(self.ops)
        for edge in (lane_from, lane_to):   # a fused add stays with its convolution
            assert edge == len(self.ops) or self.ops[edge]["op"] != "add" or self.ops[edge]["b"] not in self.unwritten
        sub = batch // lanes
        plans = {}  # (operator index, images) -> (plan, requantization): lanes share their plans

        def plan_of(index, n):
            if (index, n) in plans:
                return plans[(index, n)]
            op = self.ops[index]
            kind = op["op"]
            s, d = self.tensors[op["src"]], self.tensors[op["dst"]]
            act = eden.ACT_RELU6 if op.get("relu6") else eden.ACT_NONE
            pairs = None
            if per_channel and kind != "fc":
                w, b, w_scales = op_weights_perchannel(op, s["c"])
                q, mults, shifts = eden.make_requant_perchannel(s["scale"], s["zp"], w_scales, d["scale"], d["zp"], act,
                                                                bool(op.get("relu6")))
                pairs = (mults, shifts)
            else:
                w, b = op_weights(op, s["c"])
                q = eden.make_requant(s["scale"], s["zp"], op["w_scale"], op["w_zp"], d["scale"], d["zp"], act, bool(op.get("relu6")))
            w_layout = eden.W_OIHW | (eden.W_SIGNED if pairs else 0)
            d_w, d_b = eden.DeviceBuffer(host=w), eden.DeviceBuffer(host=b)
            self._keep += [d_w, d_b]
            if kind == "fc":
                plan = eden.FcPlan(n, s["c"], op["cout"], d_w, d_b, q, stream)
            else:
                desc = eden.conv_desc(n, s["c"], s["h"], s["w"], op["cout"], op["k"], op["k"], (op["stride"],) * 2, (op["pad"],) * 4,
                                      (1, 1), 1, 1, eden.NHWC, w_layout)
                plan = (eden.DwConvPlan if kind == "dw" else eden.ConvPlan)(desc, d_w, d_b, q, stream)
                if pairs:
                    plan.set_perchannel(*pairs)
            plans[(index, n)] = (plan, q)
            return plans[(index, n)]

        in_lane = lambda index: lane_from <= index < lane_to
        # An expansion (1x1 convolution, ReLU6) and the 3x3 depthwise convolution behind it as one launch, the expanded
        # tensor in LDS only: fuse_blocks is "auto" (wherever the library's measured table prefers it for the shape and
        # the images a launch covers) or the operator indices of the expansions to fuse.
        self.in_lds = set()   # expanded tensors that are never stored
        self.fused_blocks = []
        for index in range(len(self.ops) - 1):
            op, nxt = self.ops[index], self.ops[index + 1]
            if not (op["op"] == "conv" and op["k"] == 1 and nxt["op"] == "dw" and nxt["src"] == op["dst"] and readers[op["dst"]] == 1
                    and in_lane(index) == in_lane(index + 1)) or not fuse_blocks:
                continue
            n = sub if in_lane(index) else batch
            if fuse_blocks == "auto":
                pw, dw = plan_of(index, n)[0], plan_of(index + 1, n)[0]
                chosen = eden.conv_dw_block_preferred(pw, dw)
            else:
                chosen = index in fuse_blocks
                assert not chosen or eden.conv_dw_block_applies(plan_of(index, n)[0], plan_of(index + 1, n)[0])
            if chosen:
                self.in_lds.add(op["dst"])
                self.fused_blocks.append(index)
        size = lambda i, n=batch: n * self.tensors[i]["h"] * self.tensors[i]["w"] * self.tensors[i]["c"]
        # Tensors the full-batch operators write live in self.buffers; those the lanes write live in the lane's own
        # buffers, sized for its share of the images (a lane's tensors must not share storage with another lane's:
        # the lanes are at different operators at any moment).
        # What the lanes write and an operator after them reads is one tensor again: it lives in self.buffers and every
        # lane writes its share of it.
        read_after = {op[k] for op in self.ops[lane_to:] for k in ("src", "a", "b") if k in op}
        if lane_to == len(self.ops):
            read_after.add(len(self.tensors) - 1)   # the logits
        made_in_lane = {op["dst"] for op in self.ops[lane_from:lane_to]} - read_after
        self.buffers = [None] * len(self.tensors)
        self.lane_buffers = [[None] * len(self.tensors) for _ in range(lanes if lane_from < lane_to else 0)]
        if pooled:
            left = dict(readers)
            left[0] += 1   # the network input keeps its storage, so that a replay reads the same image again

            def place(pool, table, first_op, last_op, n, lefts):
                for index in range(first_op, last_op):
                    op = self.ops[index]
                    if op["dst"] in self.unwritten or op["dst"] in self.in_lds:
                        continue   # its reads happen in the fused launch, which is where its inputs are handed back
                    if table is self.buffers or op["dst"] in made_in_lane:
                        table[op["dst"]] = pool.request(eden.POOL_INTER_REUSE, size(op["dst"], n))
                    reads = [op[k] for k in ("src", "a", "b") if k in op and op[k] not in self.unwritten and op[k] not in self.in_lds]
                    if op["op"] == "add" and op["b"] in self.unwritten:
                        reads.append(self.ops[index - 1]["src"])   # the fused launch reads the projection's input
                    if op["op"] == "dw" and op["src"] in self.in_lds:
                        reads.append(self.ops[index - 1]["src"])   # the fused launch reads the expansion's input
                    for t in reads:
                        lefts[t] -= 1
                        if lefts[t] == 0 and table[t] is not None:   # (a lane hands back only what it owns)
                            pool.reset_inter(table[t])

            self.pool = eden.BufferPool()
            self.buffers[0] = self.pool.request(eden.POOL_INTER_NEW, size(0))
            place(self.pool, self.buffers, 0, lane_from, batch, left)
            # the tensors that leave the lanes are placed before the lanes start and stay until their readers are done
            for t in sorted(read_after & {op["dst"] for op in self.ops[lane_from:lane_to]}):
                self.buffers[t] = self.pool.request(eden.POOL_INTER_REUSE, size(t))
            self.lane_pools = []
            after = dict(left)
            for table in self.lane_buffers:
                pool = eden.BufferPool()
                after = dict(left)
                place(pool, table, lane_from, lane_to, sub, after)
                self.lane_pools.append(pool)
            place(self.pool, self.buffers, lane_to, len(self.ops), batch, after)
            self.pool_bytes = self.pool.assign() + sum(pool.assign() for pool in self.lane_pools)
        else:
            for i in range(len(self.tensors)):
                if i in self.in_lds:
                    continue
                if i in made_in_lane:
                    for table in self.lane_buffers:
                        table[i] = eden.DeviceBuffer(nbytes=size(i, sub))
                else:
                    self.buffers[i] = eden.DeviceBuffer(nbytes=size(i))
            self.pool_bytes = None
        def build(first_op, last_op, lane):
            """The steps of operators first_op .. last_op - 1; lane: None = on the whole batch, else that lane's share"""
            n = batch if lane is None else sub

            def view(t):
                if lane is None:
                    return self.buffers[t]
                if t in made_in_lane:
                    return self.lane_buffers[lane][t]
                return eden.BufferView(self.buffers[t], size(t, lane * sub)) if lanes > 1 else self.buffers[t]

            steps = []
            for index in range(first_op, last_op):
                op = self.ops[index]
                kind = op["op"]
                if kind == "add":
                    a, b, d = (self.tensors[op[k]] for k in ("a", "b", "dst"))
                    q_add = eden.make_add_requant(a["scale"], a["zp"], b["scale"], b["zp"], d["scale"], d["zp"])
                    if op["b"] in self.unwritten:
                        assert steps and steps[-1][0] == "plan", "a fused add and its convolution belong to the same lane"
                        plan, src, _, q = steps[-1][1]
                        steps[-1] = ("plan_add", (plan, src, view(op["a"]), view(op["dst"]), q, q_add))
                    else:
                        steps.append(("add", (view(op["a"]), view(op["b"]), view(op["dst"]), n * d["h"] * d["w"] * d["c"], q_add)))
                elif kind == "avgpool":
                    steps.append(("avgpool", (view(op["src"]), view(op["dst"]), self.tensors[op["src"]], op["k"], n)))
                elif kind == "dw" and op["src"] in self.in_lds:
                    dw, q_dw = plan_of(index, n)
                    assert steps and steps[-1][0] == "plan", "an expansion and its depthwise convolution belong to the same lane"
                    pw, src, _, q_pw = steps[-1][1]
                    steps[-1] = ("block", (pw, dw, src, view(op["dst"]), q_pw, q_dw))
                else:
                    plan, q = plan_of(index, n)
                    steps.append(("plan", (plan, view(op["src"]), None if op["dst"] in self.unwritten or op["dst"] in self.in_lds else view(op["dst"]), q)))
            return steps

        self.steps = build(0, lane_from, None)
        self.lane_steps = [build(lane_from, lane_to, lane) for lane in range(len(self.lane_buffers))]
        self.tail_steps = build(lane_to, len(self.ops), None)
        self.lanes, self.lane_from, self.lane_to = len(self.lane_buffers), lane_from, lane_to
        # lanes beyond the first run on streams of their own, forked from and joined to the caller's
        self.lane_streams = [eden.Stream() for _ in self.lane_steps[1:]]
        self.fork = eden.Event()
        self.joins = [eden.Event() for _ in self.lane_streams]
        eden.sync(stream)

    def set_input(self, x_nhwc):
        x = np.ascontiguousarray(x_nhwc, np.uint8)
        assert x.shape == (self.batch, self.image, self.image, 3)
        lib = self.eden.load()
        self.eden.check(lib.eh_h2d(self.buffers[0].ptr, x.ctypes.data, x.nbytes, None))
        self.eden.sync()

    def run(self, stream=None):
        """Enqueues every operator in order on `stream` (a raw handle or None); the lanes fork from it and join it."""
        self._enqueue(self.steps, stream)
        if not self.lane_steps:
            return self._enqueue(self.tail_steps, stream)
        if self.lane_streams:
            self.fork.record(stream)
        for side in self.lane_streams:
            self.fork.wait_on(side.h)
        # a lane's operators in one go (captured with the lanes' operators taking turns, four lanes replay a third slower)
        for lane, steps in enumerate(self.lane_steps):
            self._enqueue(steps, stream if lane == 0 else self.lane_streams[lane - 1].h)
        for side, join in zip(self.lane_streams, self.joins):
            join.record(side.h)
            join.wait_on(stream)
        self._enqueue(self.tail_steps, stream)

    def _enqueue(self, steps, stream):
        eden = self.eden
        for kind, args in steps:
            if kind == "plan":
                plan, src, dst, q = args
                plan.run(src, dst, q, stream)
            elif kind == "plan_add":
                plan, src, residual, dst, q, q_add = args
                plan.run_add(src, residual, dst, q, q_add, stream)
            elif kind == "add":
                a, b, dst, count, q = args
                eden.add_u8(a, b, dst, count, q, stream)
            elif kind == "block":
                pw, dw, src, dst, q_pw, q_dw = args
                eden.conv_dw_block_run(pw, dw, src, dst, q_pw, q_dw, stream=stream)
            else:
                src, dst, s, k, n = args
                eden.avgpool_u8(src, dst, n, s["c"], s["h"], s["w"], k, k, layout=eden.NHWC, stream=stream)

    def tensor(self, index):
        """Downloads tensor `index` as [batch, h, w, c]."""
        t = self.tensors[index]
        if self.buffers[index] is not None:
            return self.buffers[index].download((self.batch, t["h"], t["w"], t["c"]))
        share = self.batch // self.lanes
        return np.concatenate([table[index].download((share, t["h"], t["w"], t["c"])) for table in self.lane_buffers])

    def logits(self):
        return self.tensor(len(self.tensors) - 1).reshape(self.batch, -1)
