"""MobileNetV2-1.0 uint8 (BASELINE configs[4]): every operator of the GPU operator list against the oracle
evaluating the same list, bit-exact tensor by tensor, at small batches directly and at the full batch of 64 on an
input made of eight distinct oracle-evaluated images scattered over the batch positions without a period."""
import functools
import importlib

import numpy as np
import pytest

import oracle_lib as O
from harness import eden, oracle_forward, scattered_batch, to_eh_requant

mobilenet = importlib.import_module("cl-eden-kernel_amd.mobilenet")

pytestmark = pytest.mark.gpu


def assert_network_alive(ops, want, batch):
    """no operator's output has collapsed to a constant or to the clamps"""
    for op in ops:
        v = want[op["dst"]]
        assert v.std() > 8, (op["op"], op["dst"], float(v.std()))
        assert np.mean((v == 0) | (v == 255)) < 0.8, (op["op"], op["dst"])
    logits = want[-1].reshape(batch, -1)
    assert len(np.unique(logits)) > 40
    assert not np.array_equal(logits[0], logits[1])


@pytest.mark.parametrize("weights", ["minmax", "narrow"])
@pytest.mark.parametrize("fuse_add", [False, True], ids=["separate_adds", "fused_adds"])
@pytest.mark.parametrize("batch,image", [(2, 224), (3, 96)])
def test_mobilenet_v2_matches_oracle_tensor_by_tensor(batch, image, fuse_add, weights):
    print("mobilenet", batch, image, fuse_add, weights, flush=True)
    x = mobilenet.network_input(batch, image)
    tensors, ops, want = oracle_forward(x, image, weights=weights)
    if weights == "minmax":  # per-tensor min/max quantized: every weight tensor uses the whole byte range
        for op in ops:
            if "w_seed" in op:
                w, _ = mobilenet.op_weights(op, tensors[op["src"]]["c"])
                assert (w.min(), w.max()) == (0, 255)
    net = mobilenet.MobileNetV2(eden, batch, image, fuse_add=fuse_add, weights=weights)
    net.set_input(x)
    net.run()
    eden.sync()
    assert len(net.unwritten) == (10 if fuse_add else 0)  # every residual connection of the network
    for op in ops:
        i = op["dst"]
        if i in net.unwritten:  # the projection inside a fused convolution + add is never stored
            continue
        got = net.tensor(i).transpose(0, 3, 1, 2)
        assert np.array_equal(got, want[i]), (op["op"], i, tensors[i], int((got != want[i]).sum()))
    assert_network_alive(ops, want, batch)


DISTINCT = 8


@functools.lru_cache(maxsize=None)
def oracle_images(per_channel, weights):
    """the oracle's tensors for DISTINCT different images"""
    return oracle_forward(mobilenet.network_input(DISTINCT), 224, per_channel, weights)


@pytest.mark.parametrize("per_channel,weights", [(False, "minmax"), (False, "narrow"), (True, "minmax")],
                         ids=["per_tensor_minmax", "per_tensor_narrow", "per_channel_minmax"])
def test_mobilenet_v2_full_batch_64(per_channel, weights):
    """The network exactly as the benchmark builds it (batch 64, which decides tile shapes, grids and the depthwise
    tile width) on eight distinct images scattered over the 64 batch positions: every tensor of every batch position
    must equal the oracle's tensor for the image that sits there."""
    print("mobilenet batch 64", per_channel, weights, flush=True)
    batch = 64
    tensors, ops, want = oracle_images(per_channel, weights)
    where = scattered_batch(batch, DISTINCT)
    x = mobilenet.network_input(DISTINCT)[where]
    net = mobilenet.MobileNetV2(eden, batch, 224, fuse_add=True, per_channel=per_channel, weights=weights)
    net.set_input(x)
    stream = eden.Stream()
    graph = eden.Graph(stream, lambda s: net.run(s))   # as the benchmark launches it
    graph.launch(stream)
    stream.sync()
    for op in ops:
        i = op["dst"]
        if i in net.unwritten:
            continue
        got = net.tensor(i).transpose(0, 3, 1, 2)
        expect = want[i][where]
        if not np.array_equal(got, expect):
            img = int(np.argwhere((got != expect).reshape(batch, -1).any(axis=1))[0, 0])
            raise AssertionError((op["op"], i, img, int(where[img]), tensors[i], int((got[img] != expect[img]).sum())))
    assert_network_alive(ops, want, DISTINCT)


@pytest.mark.parametrize("per_channel", [False, True], ids=["per_tensor", "per_channel"])
def test_mobilenet_v2_on_pooled_buffers_batch_64(per_channel):
    """The network as the benchmark runs it: feature maps in the library's buffer pool (liveness reuse, one device
    allocation), batch 64, one graph replay; the logits at every batch position must equal the oracle's for the
    image that sits there (eight distinct images, scattered), on two replays."""
    batch = 64
    tensors, ops, want = oracle_images(per_channel, "minmax")
    where = scattered_batch(batch, DISTINCT)
    net = mobilenet.MobileNetV2(eden, batch, 224, fuse_add=True, per_channel=per_channel, pooled=True)
    assert net.pool_bytes < 0.45 * sum(batch * t["h"] * t["w"] * t["c"] for t in tensors)
    net.set_input(mobilenet.network_input(DISTINCT)[where])
    stream = eden.Stream()
    graph = eden.Graph(stream, lambda s: net.run(s))
    ref = want[-1].reshape(DISTINCT, -1)[where]
    for rep in range(2):
        graph.launch(stream)
        stream.sync()
        got = net.logits()
        assert np.array_equal(got, ref), (rep, np.argwhere((got != ref).any(axis=1)).ravel().tolist())


@pytest.mark.parametrize("pooled", [False, True], ids=["own_buffers", "pooled"])
@pytest.mark.parametrize("lanes,lane_from,lane_to", [(2, None, None), (4, None, None), (2, 13, None), (2, 6, 50), (2, 0, 39)],
                         ids=["two_lanes", "four_lanes", "late_lanes", "middle_lanes", "early_lanes"])
def test_mobilenet_v2_image_lanes_and_fused_blocks_match_oracle(lanes, lane_from, lane_to, pooled):
    """The operator list as chains of image shares on streams of their own (all of it, or a range of its operators with
    full-batch operators before and after), with every expansion + depthwise pair the fused kernel fits run as one
    launch: every stored tensor (own buffers) or the logits (pooled, on two replays of the captured graph) against
    the oracle, on eight distinct images."""
    batch = DISTINCT
    tensors, ops, want = oracle_images(False, "minmax")
    blocks = tuple(i for i in range(len(ops) - 1) if ops[i]["op"] == "conv" and ops[i]["k"] == 1 and ops[i + 1]["op"] == "dw")
    assert len(blocks) == 16
    net = mobilenet.MobileNetV2(eden, batch, 224, fuse_add=True, pooled=pooled, lanes=lanes, lane_from=lane_from, lane_to=lane_to,
                                fuse_blocks=blocks)
    assert net.lanes == lanes and len(net.fused_blocks) == 16 and len(net.in_lds) == 16
    net.set_input(mobilenet.network_input(DISTINCT))
    stream = eden.Stream()
    graph = eden.Graph(stream, lambda s: net.run(s))
    for rep in range(2):
        graph.launch(stream)
        stream.sync()
        assert np.array_equal(net.logits(), want[-1].reshape(DISTINCT, -1)), rep
    if not pooled:
        for op in ops:
            i = op["dst"]
            if i in net.unwritten or i in net.in_lds:
                continue
            got = net.tensor(i).transpose(0, 3, 1, 2)
            assert np.array_equal(got, want[i]), (op["op"], i, tensors[i], int((got != want[i]).sum()))
    # outside a graph: the lanes' streams fork from and join the caller's
    net.set_input(mobilenet.network_input(DISTINCT)[::-1].copy())
    net.run(stream.h)
    stream.sync()
    assert np.array_equal(net.logits(), want[-1].reshape(DISTINCT, -1)[::-1])


def test_mobilenet_v2_as_the_benchmark_runs_it_batch_64():
    """Batch 64, pooled feature maps, two lanes of 32 images, the pairs the library's table prefers fused: the logits at
    every batch position against the oracle's for the image that sits there."""
    batch = 64
    tensors, ops, want = oracle_images(False, "minmax")
    where = scattered_batch(batch, DISTINCT)
    net = mobilenet.MobileNetV2(eden, batch, 224, fuse_add=True, pooled=True, lanes=2, fuse_blocks="auto")
    assert net.lanes == 2 and 4 <= len(net.fused_blocks) < 16
    net.set_input(mobilenet.network_input(DISTINCT)[where])
    stream = eden.Stream()
    graph = eden.Graph(stream, lambda s: net.run(s))
    ref = want[-1].reshape(DISTINCT, -1)[where]
    for rep in range(2):
        graph.launch(stream)
        stream.sync()
        got = net.logits()
        assert np.array_equal(got, ref), (rep, np.argwhere((got != ref).any(axis=1)).ravel().tolist())


def test_mobilenet_v2_graph_replay_equals_eager():
    """The whole operator list captured once; every replay (with eager work between replays) gives the eager logits."""
    batch, image = 2, 96
    x = mobilenet.network_input(batch, image)
    net = mobilenet.MobileNetV2(eden, batch, image, fuse_add=True)
    net.set_input(x)
    net.run()
    eden.sync()
    eager = net.logits().copy()
    stream = eden.Stream()
    graph = eden.Graph(stream, lambda s: net.run(s))
    lib = eden.load()
    for rep in range(3):
        eden.check(lib.eh_memset(net.buffers[-1].ptr, 0, eager.size, None))
        eden.sync()
        graph.launch(stream)
        stream.sync()
        assert np.array_equal(net.logits(), eager), rep
        net.run()           # eager work between the replays
        eden.sync()


@pytest.mark.parametrize("batch,image", [(2, 224), (3, 96)])
def test_mobilenet_v2_per_channel_weights_matches_oracle_tensor_by_tensor(batch, image):
    """The same network with int8 weights and one scale per output channel in every convolution and depthwise
    convolution (uint8 tensors, residual adds inside the projection convolutions)."""
    print("mobilenet per-channel", batch, image, flush=True)
    x = mobilenet.network_input(batch, image)
    tensors, ops, want = oracle_forward(x, image, per_channel=True)
    net = mobilenet.MobileNetV2(eden, batch, image, fuse_add=True, per_channel=True)
    net.set_input(x)
    net.run()
    eden.sync()
    assert len(net.unwritten) == 10
    for op in ops:
        i = op["dst"]
        if i in net.unwritten:
            continue
        got = net.tensor(i).transpose(0, 3, 1, 2)
        assert np.array_equal(got, want[i]), (op["op"], i, tensors[i], int((got != want[i]).sum()))
    assert_network_alive(ops, want, batch)
