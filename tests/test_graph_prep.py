"""Host-side graph preparation (no GPU): the rewrite of an RGB stem for the device -- channels padded to 4, stride-2
windows read as windows over 2 x 2 pixel blocks, odd windows and odd front paddings grown by taps of zero weight --
leaves the integer convolution unchanged.  Both graphs are evaluated by the CPU oracle."""
import numpy as np
import pytest

from nncase_amd import netbuilder as nb
from oracle import netref

f32 = np.float32


def single_conv_graph(rng, h, w, cin, cout, kh, kw, stride, padding):
    q_in = nb.QNode("input", (), "input", (3, f32(1 / 255)), (cin, h, w))
    oh = (h + sum(padding[0]) - kh) // stride[0] + 1
    ow = (w + sum(padding[1]) - kw) // stride[1] + 1
    conv = nb.QNode("conv", (0,), "stem", (7, f32(0.05)), (cout, oh, ow),
                    weights=rng.integers(0, 256, (cout, cin, kh, kw), dtype=np.uint8), w_qp=(121, f32(0.004)),
                    bias=rng.integers(-500, 500, cout).astype(np.int32), stride=stride, padding=padding, clamp=(0.0, 6.0))
    return nb.QuantGraph([q_in, conv], (h, w, cin), None)


@pytest.mark.parametrize("k,stride,pad,hw,expect", [
    ((3, 3), (2, 2), ((1, 1), (1, 1)), (16, 20), "s2d"),      # MobileNetV2's stem: odd window, odd front padding
    ((3, 3), (2, 2), ((0, 1), (0, 1)), (16, 20), "s2d"),      # TF 'SAME' at an even size: the zero tap goes behind
    ((6, 6), (2, 2), ((2, 2), (2, 2)), (12, 16), "s2d"),      # YOLOv5's stem
    ((5, 5), (2, 2), ((2, 2), (2, 2)), (14, 10), "s2d"),
    ((7, 7), (2, 2), ((3, 3), (3, 3)), (18, 22), "s2d"),
    ((4, 2), (2, 2), ((1, 1), (0, 0)), (10, 12), "s2d"),
    ((3, 3), (2, 2), ((1, 1), (1, 1)), (15, 20), "none"),     # odd height: 3x3 stays with the kernel for few channels
    ((6, 6), (2, 2), ((2, 2), (2, 2)), (13, 16), "fold2"),    # odd height: only the width folds
    ((5, 5), (1, 1), ((2, 2), (2, 2)), (9, 9), "padc"),
    ((3, 3), (1, 1), ((1, 1), (1, 1)), (9, 9), "none"),
])
@pytest.mark.parametrize("cin", [1, 3])
def test_stem_rewrite_keeps_the_integer_result(k, stride, pad, hw, expect, cin):
    rng = np.random.default_rng(k[0] * 100 + hw[0] + cin)
    g = single_conv_graph(rng, hw[0], hw[1], cin, 8, k[0], k[1], stride, pad)
    g2 = nb.pad_small_channel_convs(g)
    ops = [n.op for n in g2.nodes]
    assert {"s2d": "s2d" in ops, "fold2": "fold2" in ops, "padc": ops == ["input", "padc", "conv"], "none": ops == ["input", "conv"]}[expect], ops
    conv2 = g2.nodes[-1]
    assert conv2.out_shape == g.nodes[-1].out_shape and conv2.macs == g.nodes[-1].macs
    if expect == "s2d":
        assert tuple(conv2.stride) == (1, 1) and conv2.weights.shape[1] == 16
    x = rng.random((2, hw[0], hw[1], cin), dtype=f32)
    want, outs = netref.run_integer(g, x, keep_all=True)
    got, outs2 = netref.run_integer(g2, x, keep_all=True)
    assert np.array_equal(outs[-1], outs2[-1])
    assert np.array_equal(want.view(np.uint32), got.view(np.uint32))
