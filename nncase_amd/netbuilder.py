"""Builds the quantised graphs of the benchmark configurations on the host and binds them to
a resident `hip` function.

What the reference's compiler does for a "u8/u8" model and this module reproduces:
  * fold BatchNorm into the preceding conv: scale = gamma / sqrt(var + eps),
    bias = beta - gamma * mean / sqrt(var + eps)   (src/Nncase.Passes/Rules/Neutral/BatchNormToBinary.cs:23-50)
  * ReLU6 -> Clamp(0, 6) fused into the conv as fused_clamp, applied to the float value before
    the Quantize                                       (ReluToClamp.cs:39-48, FuseClampConv2D.cs:22-38)
  * PTQ: running finite min/max of every activation over the calibration set (NoClip), the
    calibrator's FixUpRange, GetQuantParam(UnsignedMode, 8 bits)
                                                       (Quantizer.cs:358-408, QuantUtility.cs:41-97)
  * per-tensor asymmetric u8 weights, int32 bias with quant param (0, sx * sw)
                                                       (QLinearConv.cs:73)
The float forward pass used for calibration runs on the host (numpy); it plays the role of the
reference's Evaluator during calibration and is not part of the timed path.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from . import quant
from . import runtime as rt
from .runtime import Context, Function, qp

f32 = np.float32
FULL_CLAMP = (-rt.FLT_MAX, rt.FLT_MAX)


# --------------------------------------------------------------------------------------------- float graph
@dataclass
class Node:
    op: str                      # "input" | "conv" | "add" | "gap" | "swish" | "concat" | "resize" | "maxpool"
    inputs: Tuple[int, ...] = ()
    name: str = ""
    # conv
    weights: Optional[np.ndarray] = None   # OIHW float32 (BN already folded)
    bias: Optional[np.ndarray] = None      # float32 [O]
    stride: Tuple[int, int] = (1, 1)
    padding: Tuple[Tuple[int, int], Tuple[int, int]] = ((0, 0), (0, 0))
    groups: int = 1
    clamp: Tuple[float, float] = FULL_CLAMP
    # resize: output = input extent * scale (nearest, asymmetric coordinates, floor); maxpool: (kernel, stride, pad)
    scale: int = 2
    pool: Tuple[int, int, int] = (5, 1, 2)


@dataclass
class FloatGraph:
    nodes: List[Node] = field(default_factory=list)
    input_shape: Tuple[int, int, int] = (224, 224, 3)  # H, W, C (NHWC at the boundary)
    outputs: Optional[List[int]] = None                 # node ids returned (default: the last node)

    def add(self, node: Node) -> int:
        self.nodes.append(node)
        return len(self.nodes) - 1


def _kaiming(rng, shape):
    fan_in = shape[1] * shape[2] * shape[3]
    return (rng.standard_normal(shape) * np.sqrt(2.0 / fan_in)).astype(f32)


def _conv_bn(rng, g: FloatGraph, src: int, cin: int, cout: int, k: int, stride: int, groups: int, relu6: bool, name: str) -> int:
    w = _kaiming(rng, (cout, cin // groups, k, k))
    gamma = rng.uniform(0.8, 1.2, cout).astype(f32)
    beta = (rng.standard_normal(cout) * 0.1).astype(f32)
    mean = (rng.standard_normal(cout) * 0.1).astype(f32)
    var = rng.uniform(0.8, 1.2, cout).astype(f32)
    scale = gamma / np.sqrt(var + f32(1e-5))
    w = (w * scale.reshape(-1, 1, 1, 1)).astype(f32)
    b = (beta - gamma * mean / np.sqrt(var + f32(1e-5))).astype(f32)
    p = (k - 1) // 2
    return g.add(Node("conv", (src,), name, w, b, (stride, stride), ((p, p), (p, p)), groups,
                      (0.0, 6.0) if relu6 else FULL_CLAMP))


def mobilenet_v2(seed: int = 2, num_classes: int = 1000, input_hw: int = 224) -> FloatGraph:
    """MobileNetV2, width 1.0, torchvision layer table, random Kaiming weights, BN folded."""
    rng = np.random.default_rng(seed)
    g = FloatGraph(input_shape=(input_hw, input_hw, 3))
    x = g.add(Node("input", name="input"))
    x = _conv_bn(rng, g, x, 3, 32, 3, 2, 1, True, "stem")
    cin = 32
    cfg = [(1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2), (6, 320, 1, 1)]
    bi = 0
    for t, c, n, s in cfg:
        for i in range(n):
            stride = s if i == 0 else 1
            inp = x
            hidden = cin * t
            if t != 1:
                x = _conv_bn(rng, g, x, cin, hidden, 1, 1, 1, True, f"b{bi}.expand")
            x = _conv_bn(rng, g, x, hidden, hidden, 3, stride, hidden, True, f"b{bi}.dw")
            x = _conv_bn(rng, g, x, hidden, c, 1, 1, 1, False, f"b{bi}.project")
            if stride == 1 and cin == c:
                x = g.add(Node("add", (inp, x), f"b{bi}.add"))
            cin = c
            bi += 1
    x = _conv_bn(rng, g, x, cin, 1280, 1, 1, 1, True, "head")
    x = g.add(Node("gap", (x,), "pool"))
    w = (rng.standard_normal((num_classes, 1280, 1, 1)) * 0.01).astype(f32)
    g.add(Node("conv", (x,), "fc", w, np.zeros(num_classes, f32)))
    return g


def conv_block(seed: int = 1) -> FloatGraph:
    """1x1 64->144, 3x3 depthwise, 1x1 144->64 on 56x56, ReLU6 after each."""
    rng = np.random.default_rng(seed)
    g = FloatGraph(input_shape=(56, 56, 64))
    x = g.add(Node("input", name="input"))
    for name, cin, cout, k, groups in (("pw1", 64, 144, 1, 1), ("dw", 144, 144, 3, 144), ("pw2", 144, 64, 1, 1)):
        w = _kaiming(rng, (cout, cin // groups, k, k))
        b = (rng.standard_normal(cout) * 0.01).astype(f32)
        p = (k - 1) // 2
        x = g.add(Node("conv", (x,), name, w, b, (1, 1), ((p, p), (p, p)), groups, (0.0, 6.0)))
    return g


def yolov5s(seed: int = 4, input_hw: int = 640, num_outputs: int = 255) -> FloatGraph:
    """YOLOv5s-style CSP backbone + PAN neck + detect head (v6 layer table, width 0.5, depth 0.33),
    random Kaiming weights, BN folded, SiLU after every Conv block, three detect convolutions."""
    rng = np.random.default_rng(seed)
    g = FloatGraph(input_shape=(input_hw, input_hw, 3))
    x = g.add(Node("input", name="input"))
    counter = [0]

    def conv(src, cin, cout, k, s, pad=None):
        i = counter[0]
        counter[0] += 1
        y = _conv_bn(rng, g, src, cin, cout, k, s, 1, False, f"conv{i}")
        if pad is not None:
            g.nodes[y].padding = ((pad, pad), (pad, pad))
        return g.add(Node("swish", (y,), f"conv{i}.silu"))

    def c3(src, c1, c2, n, shortcut=True):
        c_ = c2 // 2
        a = conv(src, c1, c_, 1, 1)
        for _ in range(n):
            y = conv(conv(a, c_, c_, 1, 1), c_, c_, 3, 1)
            a = g.add(Node("add", (a, y), f"bottleneck{counter[0]}.add")) if shortcut else y
        b = conv(src, c1, c_, 1, 1)
        return conv(g.add(Node("concat", (a, b), f"c3_{counter[0]}.cat")), 2 * c_, c2, 1, 1)

    def sppf(src, c1, c2):
        c_ = c1 // 2
        x1 = conv(src, c1, c_, 1, 1)
        y1 = g.add(Node("maxpool", (x1,), "sppf.mp1"))
        y2 = g.add(Node("maxpool", (y1,), "sppf.mp2"))
        y3 = g.add(Node("maxpool", (y2,), "sppf.mp3"))
        return conv(g.add(Node("concat", (x1, y1, y2, y3), "sppf.cat")), 4 * c_, c2, 1, 1)

    x = conv(x, 3, 32, 6, 2, pad=2)
    x = conv(x, 32, 64, 3, 2)
    x = c3(x, 64, 64, 1)
    x = conv(x, 64, 128, 3, 2)
    p3 = c3(x, 128, 128, 2)
    x = conv(p3, 128, 256, 3, 2)
    p4 = c3(x, 256, 256, 3)
    x = conv(p4, 256, 512, 3, 2)
    x = c3(x, 512, 512, 1)
    x = sppf(x, 512, 512)
    n10 = conv(x, 512, 256, 1, 1)
    x = g.add(Node("resize", (n10,), "up1"))
    x = c3(g.add(Node("concat", (x, p4), "cat_p4")), 512, 256, 1, False)
    n14 = conv(x, 256, 128, 1, 1)
    x = g.add(Node("resize", (n14,), "up2"))
    o3 = c3(g.add(Node("concat", (x, p3), "cat_p3")), 256, 128, 1, False)
    x = conv(o3, 128, 128, 3, 2)
    o4 = c3(g.add(Node("concat", (x, n14), "cat_n14")), 256, 256, 1, False)
    x = conv(o4, 256, 256, 3, 2)
    o5 = c3(g.add(Node("concat", (x, n10), "cat_n10")), 512, 512, 1, False)
    heads = []
    for name, src, c in (("detect_p3", o3, 128), ("detect_p4", o4, 256), ("detect_p5", o5, 512)):
        w = (rng.standard_normal((num_outputs, c, 1, 1)) * np.sqrt(1.0 / c)).astype(f32)
        b = (rng.standard_normal(num_outputs) * 0.1).astype(f32)
        heads.append(g.add(Node("conv", (src,), name, w, b)))
    g.outputs = heads
    return g


# --------------------------------------------------------------------------------------------- host float pass
def _conv_float(x: np.ndarray, n: Node) -> np.ndarray:
    """NCHW float conv via im2col + matmul (calibration only)."""
    b, c, h, w = x.shape
    oc, gic, kh, kw = n.weights.shape
    (ph0, ph1), (pw0, pw1) = n.padding
    sh, sw = n.stride
    xp = np.pad(x, ((0, 0), (0, 0), (ph0, ph1), (pw0, pw1)))
    oh = (h + ph0 + ph1 - kh) // sh + 1
    ow = (w + pw0 + pw1 - kw) // sw + 1
    if n.groups == c and gic == 1 and oc == c:  # depthwise
        out = np.zeros((b, c, oh, ow), f32)
        for ky in range(kh):
            for kx in range(kw):
                out += xp[:, :, ky:ky + (oh - 1) * sh + 1:sh, kx:kx + (ow - 1) * sw + 1:sw] * n.weights[:, 0, ky, kx].reshape(1, -1, 1, 1)
    else:
        assert n.groups == 1
        cols = np.empty((b, gic, kh, kw, oh, ow), f32)
        for ky in range(kh):
            for kx in range(kw):
                cols[:, :, ky, kx] = xp[:, :, ky:ky + (oh - 1) * sh + 1:sh, kx:kx + (ow - 1) * sw + 1:sw]
        out = np.einsum("ok,bkp->bop", n.weights.reshape(oc, -1), cols.reshape(b, gic * kh * kw, oh * ow), optimize=True)
        out = out.reshape(b, oc, oh, ow).astype(f32)
    out += n.bias.reshape(1, -1, 1, 1)
    return np.clip(out, n.clamp[0], n.clamp[1]).astype(f32)


def float_forward(g: FloatGraph, x_nhwc: np.ndarray) -> List[np.ndarray]:
    """All node outputs (NCHW float32) for a batch of NHWC float32 inputs."""
    outs: List[np.ndarray] = []
    for n in g.nodes:
        if n.op == "input":
            y = np.ascontiguousarray(np.asarray(x_nhwc, f32).transpose(0, 3, 1, 2))
        elif n.op == "conv":
            y = _conv_float(outs[n.inputs[0]], n)
        elif n.op == "add":
            y = outs[n.inputs[0]] + outs[n.inputs[1]]
        elif n.op == "gap":
            y = outs[n.inputs[0]].mean(axis=(2, 3), keepdims=True).astype(f32)
        elif n.op == "swish":
            v = outs[n.inputs[0]]
            y = (v / (1 + np.exp(-v))).astype(f32)
        elif n.op == "concat":
            y = np.concatenate([outs[j] for j in n.inputs], axis=1)
        elif n.op == "resize":
            y = outs[n.inputs[0]].repeat(n.scale, axis=2).repeat(n.scale, axis=3)
        elif n.op == "maxpool":
            k, st, p = n.pool
            v = np.pad(outs[n.inputs[0]], ((0, 0), (0, 0), (p, p), (p, p)), constant_values=0.0)  # the reference folds 0 in for padding
            y = np.lib.stride_tricks.sliding_window_view(v, (k, k), axis=(2, 3))[:, :, ::st, ::st].max(axis=(-1, -2)).astype(f32)
        else:
            raise ValueError(n.op)
        outs.append(y)
    return outs


# --------------------------------------------------------------------------------------------- quantised graph
@dataclass
class QNode:
    op: str
    inputs: Tuple[int, ...]
    name: str
    out_qp: Tuple[int, np.float32]          # (zero_point, scale) of this node's u8 output
    out_shape: Tuple[int, int, int]          # C, H, W per image
    weights: Optional[np.ndarray] = None     # OIHW uint8
    w_qp: Optional[Tuple[int, np.float32]] = None
    bias: Optional[np.ndarray] = None        # int32
    stride: Tuple[int, int] = (1, 1)
    padding: Tuple[Tuple[int, int], Tuple[int, int]] = ((0, 0), (0, 0))
    groups: int = 1
    clamp: Tuple[float, float] = FULL_CLAMP
    lut: Optional[np.ndarray] = None         # "lut": 256-entry byte table Q(f(DQ(.)))
    resize_modes: Tuple[int, int] = (rt.RESIZE_ASYMMETRIC, rt.NEAREST_FLOOR)   # "resize"
    pool: Tuple[int, int, int] = (5, 1, 2)   # "maxpool": kernel, stride, pad
    model_k: Optional[int] = None            # "conv" whose weights were padded for the device: the model's own reduction length

    @property
    def macs(self) -> int:
        """Multiply-accumulates of the model's conv per image (padding taps and channels added for the device not counted)."""
        oc, gic, kh, kw = self.weights.shape
        return oc * self.out_shape[1] * self.out_shape[2] * (self.model_k if self.model_k is not None else gic * kh * kw)


@dataclass
class QuantGraph:
    """u8/u8 graph: float32 NHWC input -> Quantize -> u8 nodes -> Dequantize -> float32 output(s)."""
    nodes: List[QNode]
    input_shape: Tuple[int, int, int]
    outputs: Optional[List[int]] = None      # node ids that are dequantised and returned (default: the last node)

    @property
    def output_nodes(self) -> List[int]:
        return list(self.outputs) if self.outputs else [len(self.nodes) - 1]

    @property
    def macs_per_image(self) -> Dict[str, int]:
        dense = dw = 0
        for n in self.nodes:
            if n.op != "conv":
                continue
            m = n.macs
            if n.groups > 1 and n.weights.shape[1] == 1:
                dw += m
            else:
                dense += m
        return {"dense": dense, "depthwise": dw}


def quantize_graph(g: FloatGraph, calib_nhwc: np.ndarray, calib_batch: int = 8) -> QuantGraph:
    """Per-tensor PTQ with min/max (NoClip) calibration over `calib_nhwc`."""
    ranges: List[Optional[Tuple[np.float32, np.float32]]] = [None] * len(g.nodes)
    shapes: List[Tuple[int, int, int]] = [None] * len(g.nodes)
    for s in range(0, len(calib_nhwc), calib_batch):
        outs = float_forward(g, calib_nhwc[s:s + calib_batch])
        for i, y in enumerate(outs):
            r = quant.range_of(y)
            ranges[i] = r if ranges[i] is None else quant.union(ranges[i], r)
            shapes[i] = tuple(y.shape[1:])
    qnodes: List[QNode] = []
    for i, n in enumerate(g.nodes):
        zp, sc = quant.get_quant_param(quant.calib_fixup_range(ranges[i]), 8, quant.QuantMode.UnsignedMode)
        qn = QNode(n.op, n.inputs, n.name, (zp, sc), shapes[i])
        if n.op == "conv":
            wq, zw, sw = quant.quantize_weights(n.weights)
            sx = qnodes[n.inputs[0]].out_qp[1]
            bscale = f32(sx) * f32(sw)  # bias quant param is (0, sx * sw)
            qn.weights, qn.w_qp = wq, (zw, sw)
            qn.bias = np.clip(np.rint(n.bias / bscale), -2 ** 31, 2 ** 31 - 1).astype(np.int32)
            qn.stride, qn.padding, qn.groups, qn.clamp = n.stride, n.padding, n.groups, n.clamp
        elif n.op == "swish":
            # Dequantize -> swish -> Quantize of a u8 tensor is a byte table; the library evaluates it
            # with the CPU kernels' fp32 operations
            qn.op = "lut"
            src_qp = qnodes[n.inputs[0]].out_qp
            qn.lut = rt.make_unary_lut(rt.LUT_SWISH, qp(*src_qp), qp(zp, sc))
        elif n.op == "maxpool":
            qn.pool = n.pool
        elif n.op == "resize":
            assert shapes[i][1] == shapes[n.inputs[0]][1] * n.scale
        qnodes.append(qn)
    return pad_small_channel_convs(QuantGraph(qnodes, g.input_shape, g.outputs))


def _even_window(k: int, p0: int, size: int, out: int):
    """A stride-2 window of k taps with p0 padded positions in front, as an even window whose front padding is even
    too: (taps to prepend, taps to append, front padding, back padding), the added taps carrying zero weights and the
    back padding being what makes the output extent `out` again.  None when no such window exists."""
    front = p0 % 2                      # an odd front padding: one more (zero) tap in front
    back = (k + front) % 2              # then an odd window: one more behind
    k2, p0 = k + front + back, p0 + front
    p1 = 2 * (out - 1) + k2 - size - p0
    return None if p1 < 0 or p1 % 2 else (front, back, p0, p1)


def pad_small_channel_convs(qg: QuantGraph) -> QuantGraph:
    """A dense conv over fewer than 4 input channels (an RGB stem) would gather single bytes.  Its input is padded to
    4 channels ("padc": zero-filled 4th channel) and its weights with the weight zero point, which contributes
    (w - zw) = 0 whatever the padded byte is: the integer result is unchanged and the conv reads whole dwords.  Stems
    of stride 2 go further and read 2 x 2 pixel blocks as 16-channel pixels (below); 3x3 windows of stride 1 are left
    to the kernel for few input channels."""
    nodes: List[QNode] = []
    remap: Dict[int, int] = {}
    for i, n in enumerate(qg.nodes):
        n = QNode(**{**n.__dict__, "inputs": tuple(remap[j] for j in n.inputs)})
        small = n.op == "conv" and n.groups == 1 and n.weights.shape[1] < 4
        if small:
            src = nodes[n.inputs[0]]
            c, h, w = src.out_shape
            kh, kw = n.weights.shape[2:]
            (ph0, ph1), (pw0, pw1) = n.padding
            ev = (_even_window(kh, ph0, h, n.out_shape[1]), _even_window(kw, pw0, w, n.out_shape[2])) \
                if tuple(n.stride) == (2, 2) and h % 2 == 0 and w % 2 == 0 else (None, None)
        if small and (n.weights.shape[2:] != (3, 3) or None not in ev):
            nodes.append(QNode("padc", (n.inputs[0],), n.name + ".pad4", src.out_qp, (4, h, w)))
            wpad = np.full((n.weights.shape[0], 4) + n.weights.shape[2:], n.w_qp[0], np.uint8)
            wpad[:, :c] = n.weights
            n.model_k = int(np.prod(n.weights.shape[1:]))
            n.weights, n.inputs = wpad, (len(nodes) - 1,)
            if None not in ev:
                # Stride 2 (odd windows and odd front paddings first grow by taps of zero weight): every 2 x 2 block of
                # 4-channel pixels becomes one 16-channel pixel of the
                # half-size image ("s2d": pack by lanes (2, 2, 4) on (H, W, C), channel order (dy, dx, c)), and the conv
                # becomes one of stride 1 over half the window in both directions:
                # out(y, x) = sum over ky', kx', (dy, dx, c) of in[2 (y + ky' - ph / 2) + dy][2 (x + kx' - pw / 2) + dx][c]
                #             w[2 ky' + dy][2 kx' + dx][c].  The loader then fetches 16 bytes per tap and computes a quarter
                # as many tap addresses; the padding is whole blocks, filled with the input's zero point as before.
                (fh, bh, ph0, ph1), (fw, bw, pw0, pw1) = ev
                wpad = np.pad(wpad, ((0, 0), (0, 0), (fh, bh), (fw, bw)), constant_values=n.w_qp[0])
                kh, kw = wpad.shape[2:]
                nodes[-1] = QNode("s2d", nodes[-1].inputs, n.name + ".s2d", src.out_qp, (16, h // 2, w // 2))
                wf = np.empty((wpad.shape[0], 16, kh // 2, kw // 2), np.uint8)
                for dy in range(2):
                    for dx in range(2):
                        wf[:, (dy * 2 + dx) * 4:(dy * 2 + dx) * 4 + 4] = wpad[:, :, dy::2, dx::2]
                n.weights = wf
                n.stride = (1, 1)
                n.padding = ((ph0 // 2, ph1 // 2), (pw0 // 2, pw1 // 2))
            elif n.stride[1] == 2 and kw % 2 == 0 and w % 2 == 0 and pw0 % 2 == 0 and pw1 % 2 == 0:
                # Stride 2 along the width only: two neighbouring 4-channel pixels are one 8-channel pixel of the
                # half-width image in the same NHWC bytes ("fold2": nothing moves), and the conv becomes one of stride 1
                # along the width over half as many taps.
                nodes.append(QNode("fold2", (len(nodes) - 1,), n.name + ".fold2", src.out_qp, (8, h, w // 2)))
                wf = np.empty((wpad.shape[0], 8, kh, kw // 2), np.uint8)
                for dx in range(2):
                    wf[:, dx * 4:dx * 4 + 4] = wpad[:, :, :, dx::2]
                n.weights, n.inputs = wf, (len(nodes) - 1,)
                n.stride = (n.stride[0], 1)
                n.padding = ((ph0, ph1), (pw0 // 2, pw1 // 2))
        nodes.append(n)
        remap[i] = len(nodes) - 1
    outs = None if qg.outputs is None else [remap[j] for j in qg.outputs]
    return QuantGraph(nodes, qg.input_shape, outs)


# --------------------------------------------------------------------------------------------- device binding
# Where a pointwise pair replaces its two convolutions: while the weight bytes its workgroups stream between them
# (pixel tiles x both weight tensors) stay small, and while all its workgroups (one per 16 pixels and channel range) are
# resident at once.  Measured on MobileNetV2: every pair within these limits is quicker than its two launches at
# batches 1 and 2 (0.215 -> 0.184 ms per image at batch 1); beyond them the separate kernels win.
PAIR_STREAM_LIMIT = 4 << 20
PAIR_MAX_PIXEL_TILES = 1024
# A depthwise convolution in front joins the pair while it has few channels: a workgroup computes its 16 pixels of it
# alone, about 50 ns per 16 channels, against the 3.5 us of the separate launch it saves.
PAIR_FRONT_MAX_CHANNELS = 256


class HipModel:
    """A QuantGraph resident on the device: packed weights, one HBM buffer per tensor, and the
    operator list recorded in a `hip` function.  run() = upload input, invoke, download output.

    lanes > 1 splits the batch into that many equal image ranges and records the whole operator list once per
    range, each on its own lane of the function: a captured function then replays the lanes on concurrent
    streams, so one lane's launch gaps and tail waves are filled by the other's kernels.  Every tensor keeps
    its full-batch NHWC buffer (a lane works on its image range of it) and the lanes share the packed weights,
    so results are bit-identical to lanes == 1."""

    def __init__(self, ctx: Context, qg: QuantGraph, batch: int, capture_graph: bool = True, fuse_residual: bool = True,
                 lanes: int = 1, fuse_blocks=True, fuse_pairs=True):
        if lanes < 1 or lanes > rt.MAX_LANES or batch % lanes:
            raise ValueError(f"lanes={lanes} must be in 1..{rt.MAX_LANES} and divide the batch ({batch})")
        self.ctx, self.qg, self.batch, self.lanes = ctx, qg, batch, lanes
        bl = batch // lanes                      # images per lane
        h, w, c = qg.input_shape
        self.in_count = batch * h * w * c
        self.input_f32 = ctx.alloc(lanes * self._lane_stride(self.in_count // lanes * 4))
        self.fn = Function(ctx)
        self.buffers: List[Optional[rt.DeviceBuffer]] = []
        self.weights: List[Optional[rt.Weights]] = []
        self.op_names: List[str] = []
        self.op_nodes: List[int] = []
        self.op_members: List[List[int]] = []   # graph nodes every recorded operator computes (per lane-0 operator)
        # A residual add whose second operand is a dense conv consumed by nothing else is folded into
        # that conv's epilogue (the conv's own u8 tensor is then never written).
        consumers = [0] * len(qg.nodes)
        for n in qg.nodes:
            for j in n.inputs:
                consumers[j] += 1
        # A byte-table node (swish) whose only producer is a dense conv consumed by nothing else is applied in
        # that conv's epilogue; a residual add can then still be folded behind it.  Tensors that only exist
        # inside a fused operator are never written (materialized() is False for them).
        def dense_conv(j):
            nj = qg.nodes[j]
            return (nj.op == "conv" and not (nj.groups > 1 and nj.weights.shape[1] == 1) and nj.weights.shape[1] * nj.groups > 4
                    and consumers[j] == 1 and j not in qg.output_nodes)
        self.fused_lut: Dict[int, int] = {}    # conv node -> lut node
        self.fused_into: Dict[int, int] = {}   # conv node -> add node
        if fuse_residual:
            for i, n in enumerate(qg.nodes):
                if n.op == "lut" and n.inputs[0] == i - 1 and dense_conv(i - 1):
                    self.fused_lut[i - 1] = i
            lut_owner = {v: k for k, v in self.fused_lut.items()}
            for i, n in enumerate(qg.nodes):
                if n.op == "add":
                    a, b = n.inputs
                    conv = lut_owner.get(b, b)                      # the conv that produces operand b
                    last = self.fused_lut.get(conv, conv)           # ... and the last node fused into it so far
                    if last == b == i - 1 and a < conv and consumers[b] == 1 and b not in qg.output_nodes and \
                            (b in lut_owner or dense_conv(b)):
                        self.fused_into[conv] = i
        self.never_written = set(self.fused_into.keys()) | set(self.fused_lut.keys())
        for conv, add in self.fused_into.items():
            if conv in self.fused_lut:
                self.never_written.add(self.fused_lut[conv])
        fused_tail = set(self.fused_into.values()) | set(self.fused_lut.values())   # nodes computed in a conv's epilogue
        skip_nodes = set(fused_tail)
        # Inverted-residual blocks (1x1 conv -> 3x3 depthwise -> 1x1 conv, each consumed only by the next, optionally
        # + the block's input) run as one fused operator: the two expanded tensors then never reach HBM.
        self.blocks: Dict[int, Tuple[int, int, Optional[int]]] = {}   # expansion node -> (depthwise, projection, add or None)
        if fuse_blocks and fuse_residual:
            def pointwise(n):
                return (n.op == "conv" and n.groups == 1 and n.weights.shape[2:] == (1, 1) and tuple(n.stride) == (1, 1)
                        and tuple(map(tuple, n.padding)) == ((0, 0), (0, 0)))

            def depthwise3(n):
                return (n.op == "conv" and n.groups == n.weights.shape[0] and n.weights.shape[1:] == (1, 3, 3)
                        and tuple(n.stride) in ((1, 1), (2, 2)) and all(p in (0, 1) for pp in n.padding for p in pp))
            for i in range(len(qg.nodes) - 2):
                e, d, pr = qg.nodes[i], qg.nodes[i + 1], qg.nodes[i + 2]
                if not (pointwise(e) and depthwise3(d) and pointwise(pr)):
                    continue
                if tuple(d.inputs) != (i,) or tuple(pr.inputs) != (i + 1,) or consumers[i] != 1 or consumers[i + 1] != 1:
                    continue
                if {i, i + 1} & set(qg.output_nodes) or {i, i + 1, i + 2} & set(self.fused_lut):
                    continue
                addn = self.fused_into.get(i + 2)
                if addn is not None and (qg.nodes[addn].inputs[0] != e.inputs[0] or tuple(d.stride) != (1, 1)):
                    continue
                if not ctx.qblock_supported(e.weights.shape[1], e.weights.shape[0], pr.weights.shape[0]):
                    continue
                # Where it pays: mid-sized feature maps at batches that give the fused kernel at least 64 workgroups.
                # On large maps the three operators are bandwidth-bound kernels of their own that already run near
                # the epilogue's arithmetic cost, on 7x7 maps (and at small batches) a workgroup per tile leaves most
                # of the device idle and the three latency-bound launches are quicker.
                tiles = -(-d.out_shape[1] // 7) * -(-d.out_shape[2] // 7)        # 7x7 output tiles per image
                if fuse_blocks != "all" and not (d.out_shape[1] * d.out_shape[2] >= 196 and e.out_shape[1] * e.out_shape[2] <= 784
                                                 and (batch // lanes) * tiles >= 64):
                    continue
                self.blocks[i] = (i + 1, i + 2, addn)
        for e, (d, pr, addn) in self.blocks.items():
            self.never_written |= {e, d}
            skip_nodes |= {d, pr}
        block_members = {m for e, (d, pr, _) in self.blocks.items() for m in (e, d, pr)}
        # A dense conv (with whatever is folded into its epilogue) whose result only feeds a channel concat writes its
        # slice of the concat's tensor itself: out[p, off + c] with the concat's pixel stride.  The concat's
        # requantisation of that input, a byte table, is composed with the conv's own table (or becomes it); behind
        # a folded residual add there is no table stage, so such a conv only qualifies when the requantisation is
        # the identity.  The concat operator then skips that input, and disappears when none is left.
        self.write_through: Dict[int, Tuple[int, int, int, Optional[np.ndarray]]] = {}   # conv -> (concat, offset, stride, table)
        if fuse_residual:
            owner = {**{v: k for k, v in self.fused_lut.items()}, **{v: k for k, v in self.fused_into.items()}}
            for ci, cn in enumerate(qg.nodes):
                if cn.op != "concat":
                    continue
                ctot = sum(qg.nodes[j].out_shape[0] for j in cn.inputs)
                off = 0
                for j in cn.inputs:
                    ch = qg.nodes[j].out_shape[0]
                    conv = owner.get(j, j)
                    conv = owner.get(conv, conv)               # add -> lut -> conv
                    cnode = qg.nodes[conv]
                    last = self.fused_into.get(conv, self.fused_lut.get(conv, conv))
                    ok = (cnode.op == "conv" and last == j and consumers[j] == 1 and j not in qg.output_nodes
                          and conv not in block_members and conv not in self.write_through
                          and not (cnode.groups > 1 and cnode.weights.shape[1] == 1) and cnode.weights.shape[1] * cnode.groups > 4
                          and (conv == j or conv in self.fused_lut or conv in self.fused_into))
                    if ok:
                        table = rt.make_unary_lut(rt.LUT_REQUANT, qp(*qg.nodes[j].out_qp), qp(*cn.out_qp))
                        identity = np.array_equal(table, np.arange(256, dtype=np.uint8))
                        if conv in self.fused_into:
                            ok = identity
                            table = None
                        elif conv in self.fused_lut:
                            table = table[qg.nodes[self.fused_lut[conv]].lut]
                        elif identity:
                            table = None
                    if ok:
                        self.write_through[conv] = (ci, off, ctot, table)
                        self.never_written |= {conv, j} | ({self.fused_lut[conv]} if conv in self.fused_lut else set())
                    off += ch
        # The quantisation of the float input is done by the pack operator behind it (RGB -> RGBX or 2 x 2 blocks ->
        # 16-channel pixels in front of a stem conv) when nothing else reads the quantised RGB tensor.
        self.fused_quant: Dict[int, int] = {}                                            # pack node -> input node
        if fuse_residual:
            for i, n in enumerate(qg.nodes):
                j = n.inputs[0] if n.inputs else -1
                if n.op in ("padc", "s2d") and qg.nodes[j].op == "input" and consumers[j] == 1 and j not in qg.output_nodes:
                    self.fused_quant[i] = j
                    self.never_written.add(j)
                    skip_nodes.add(j)
        # The Dequantize of an output whose u8 tensor nothing else reads is done by the dense conv that produces it
        # (behind its folded table / add): the conv stores float32 into the output buffer.
        self.fused_dequant: Dict[int, int] = {}                                          # conv -> index into output_nodes
        if fuse_residual:
            owner = {**{v: k for k, v in self.fused_lut.items()}, **{v: k for k, v in self.fused_into.items()}}
            for oi, j in enumerate(qg.output_nodes):
                conv = owner.get(j, j)
                conv = owner.get(conv, conv)
                cnode = qg.nodes[conv]
                last = self.fused_into.get(conv, self.fused_lut.get(conv, conv))
                if (cnode.op == "conv" and last == j and consumers[j] == 0 and qg.output_nodes.count(j) == 1
                        and conv not in block_members and conv not in self.write_through
                        and not (cnode.groups > 1 and cnode.weights.shape[1] == 1) and cnode.weights.shape[1] * cnode.groups > 4
                        and (conv == j or consumers[conv] == 1)):
                    self.fused_dequant[conv] = oi
                    self.never_written |= {conv, j} | ({self.fused_lut[conv]} if conv in self.fused_lut else set())
        # A dense 1x1 convolution (with its folded table / add) whose result a second dense 1x1 convolution reads runs
        # with it as one launch where the two are latency-bound: a bottleneck's projection and the next block's
        # expansion at small batches.  Every workgroup of the pair repeats the first convolution for its 16 pixels, so
        # the weights it streams (pixel tiles x both weight tensors) bound where that still pays.
        self.pairs: Dict[int, int] = {}                                                  # first conv -> second conv
        self.pair_fronts: Dict[int, int] = {}                                            # first conv -> depthwise conv in front
        if fuse_pairs and fuse_residual:
            def pointwise1(j):
                n = qg.nodes[j]
                return (n.op == "conv" and n.groups == 1 and n.weights.shape[2:] == (1, 1) and tuple(n.stride) == (1, 1)
                        and tuple(map(tuple, n.padding)) == ((0, 0), (0, 0)) and j not in block_members
                        and j not in self.write_through and j not in self.fused_dequant)
            taken = set()
            for i, n in enumerate(qg.nodes):
                if i in taken or not pointwise1(i):
                    continue
                tail = self.fused_into.get(i, self.fused_lut.get(i, i))
                seconds = [j for j in range(tail + 1, len(qg.nodes)) if tuple(qg.nodes[j].inputs) == (tail,) and pointwise1(j)
                           and j not in self.fused_into and j not in taken]
                if not seconds:
                    continue
                j = seconds[0]
                k1, n1, n2 = n.weights.shape[1], n.weights.shape[0], qg.nodes[j].weights.shape[0]
                if not ctx.qpointwise_pair_supported(k1, n1, n2):
                    continue
                ptiles = -(-(bl * n.out_shape[1] * n.out_shape[2]) // 16)
                if fuse_pairs != "all" and (ptiles > PAIR_MAX_PIXEL_TILES or ptiles * (k1 * n1 + n1 * n2) > PAIR_STREAM_LIMIT):
                    continue
                self.pairs[i] = j
                taken |= {i, j}
                skip_nodes.add(j)
                # ... and a 3x3 depthwise convolution that only the first of the two reads is computed by the same launch,
                # 16 pixels per workgroup straight into LDS
                d = n.inputs[0]
                dn = qg.nodes[d]
                if (fuse_pairs != "nofront" and (fuse_pairs == "all" or k1 <= PAIR_FRONT_MAX_CHANNELS)
                        and dn.op == "conv" and dn.groups == dn.weights.shape[0] and dn.weights.shape[1:] == (1, 3, 3)
                        and tuple(dn.stride) in ((1, 1), (2, 2)) and consumers[d] == 1 and d not in qg.output_nodes
                        and d not in block_members and d not in self.fused_lut and d not in self.fused_into):
                    self.pair_fronts[i] = d
                    self.never_written.add(d)
                    skip_nodes.add(d)
        self.pair_objects: Dict[int, rt.QPair] = {}
        # buffers and packed weights once, shared by the lanes
        for i, n in enumerate(qg.nodes):
            cc, hh, ww = n.out_shape
            self.weights.append(None)
            if i in fused_tail:
                self.buffers.append(self.buffers[i - 1])  # written by the operator it is fused into
                continue
            if n.op == "fold2":
                self.buffers.append(self.buffers[n.inputs[0]])  # the same bytes read as half as many, twice as deep pixels
                continue
            if (i in self.blocks or i - 1 in self.blocks or i in self.write_through or i in self.fused_quant.values() or i in self.fused_dequant
                    or i in self.pair_fronts.values()):
                self.buffers.append(ctx.alloc(16))        # expanded tensors of a fused block live in LDS only; a conv
                #                                           that writes into its concat has no tensor of its own
            else:
                self.buffers.append(ctx.alloc(lanes * self._lane_stride(bl * cc * hh * ww)))
            if i in self.blocks:
                d, pr = qg.nodes[i + 1], qg.nodes[i + 2]
                self.weights[-1] = ctx.prepack_qblock(n.weights, n.bias, qp(*n.w_qp), d.weights, d.bias, qp(*d.w_qp),
                                                      pr.weights, pr.bias, qp(*pr.w_qp))
            elif n.op == "conv" and i not in block_members:
                wt = ctx.prepack_conv2d(n.weights, n.bias, qp(*n.w_qp), n.groups, expected_pixels=bl * hh * ww)
                fused_lut = self.fused_lut.get(i)
                wthru = self.write_through.get(i)
                if wthru is not None and wthru[3] is not None:
                    wt.set_post_lut(wthru[3], qp(*qg.nodes[wthru[0]].out_qp))      # own table, then the concat's requantisation
                elif fused_lut is not None:
                    wt.set_post_lut(qg.nodes[fused_lut].lut, qp(*qg.nodes[fused_lut].out_qp))
                self.weights[-1] = wt
        for a_, b_ in self.pairs.items():
            self.pair_objects[a_] = ctx.prepack_qpointwise_pair(self.weights[a_], qg.nodes[a_].weights, self.weights[b_], qg.nodes[b_].weights)
        # A global average pool that only a dense 1x1 convolution reads (a classifier's tail) is computed by that
        # convolution's launch where the library says it pays: a few rows only.
        self.pool_fronts: Dict[int, int] = {}                                            # conv -> gap node
        if fuse_pairs and fuse_residual:
            for i, n in enumerate(qg.nodes):
                readers = [j for j in range(i + 1, len(qg.nodes)) if i in qg.nodes[j].inputs]
                if n.op != "gap" or len(readers) != 1 or i in qg.output_nodes:
                    continue
                j = readers[0]
                cn = qg.nodes[j]
                if not (cn.op == "conv" and cn.groups == 1 and cn.weights.shape[2:] == (1, 1) and tuple(cn.stride) == (1, 1)
                        and tuple(map(tuple, cn.padding)) == ((0, 0), (0, 0)) and j not in block_members and j not in self.write_through
                        and j not in self.fused_into and j not in self.pairs and j not in self.pairs.values() and self.weights[j] is not None):
                    continue
                probe = rt.Conv2dArgs(bl, 1, 1, 1, 1, 1, 1, 0, 0, 0, 0, qp(*n.out_qp), qp(*cn.out_qp), cn.clamp[0], cn.clamp[1], rt.DT_U8)
                if j in self.fused_dequant:
                    probe.out_dtype, probe.dequantize_output = rt.DT_F32, 1
                src = qg.nodes[n.inputs[0]]
                if ctx.qglobal_avgpool_qconv2d_supported(self.weights[j], probe, src.out_shape[1], src.out_shape[2]):
                    self.pool_fronts[j] = i
                    self.never_written.add(i)
                    skip_nodes.add(i)
        self.outputs_f32: List[rt.DeviceBuffer] = [ctx.alloc(lanes * self._lane_stride(bl * int(np.prod(qg.nodes[j].out_shape)) * 4))
                                                    for j in qg.output_nodes]
        for lane in range(lanes):
            self.fn.set_lane(lane)
            self._record_lane(lane, bl, skip_nodes)
        self.fn.set_lane(0)
        self.output_f32 = self.outputs_f32[0]
        last = qg.nodes[qg.output_nodes[0]]
        self.out_shape = (batch,) + tuple(last.out_shape)
        self.out_count = int(np.prod(self.out_shape))
        if capture_graph:
            self.fn.capture()

    def _record_lane(self, lane: int, bl: int, skip_nodes):
        """Record the operator list for images [lane*bl, (lane+1)*bl) on the function's current lane."""
        qg = self.qg

        def B(j):                                  # this lane's image range of node j's u8 tensor
            per = bl * int(np.prod(qg.nodes[j].out_shape))
            return self.buffers[j].view(lane * self._lane_stride(per), per)

        h, w, c = qg.input_shape
        in_per = bl * h * w * c
        for i, n in enumerate(qg.nodes):
            if i in skip_nodes:
                continue
            cc, hh, ww = n.out_shape
            fused_add = self.fused_into.get(i)
            fused_lut = self.fused_lut.get(i)
            members = [i] + ([fused_lut] if fused_lut is not None else []) + ([fused_add] if fused_add is not None else [])
            if i in self.blocks:
                dn, pn, addn = self.blocks[i]
                d, pr, src = qg.nodes[dn], qg.nodes[pn], qg.nodes[n.inputs[0]]
                a = rt.QBlockArgs()
                a.batch, a.in_h, a.in_w, a.stride = bl, src.out_shape[1], src.out_shape[2], d.stride[0]
                (a.pad_h_before, a.pad_h_after), (a.pad_w_before, a.pad_w_after) = d.padding
                a.x_qp, a.expand_qp, a.dw_qp, a.y_qp = qp(*src.out_qp), qp(*n.out_qp), qp(*d.out_qp), qp(*pr.out_qp)
                a.expand_clamp_min, a.expand_clamp_max = n.clamp
                a.dw_clamp_min, a.dw_clamp_max = d.clamp
                a.clamp_min, a.clamp_max = pr.clamp
                a.add_input = int(addn is not None)
                if addn is not None:
                    a.sum_qp = qp(*qg.nodes[addn].out_qp)
                    a.sum_clamp_min, a.sum_clamp_max = FULL_CLAMP
                self.fn.add_qblock(B(n.inputs[0]), self.weights[i], B(pn), a)
                if lane == 0:
                    self.op_names.append(f"block:{n.name}" + ("+add" if addn is not None else ""))
                    self.op_nodes.append(addn if addn is not None else pn)
                    self.op_members.append([i, dn, pn] + ([addn] if addn is not None else []))
                continue
            buf = None if i in self.write_through or i in self.fused_dequant else B(i)   # (a conv that writes into its concat or
            #                                                                              the output has no tensor of its own)
            if n.op == "input":
                self.fn.add_quantize(self.input_f32.view(lane * self._lane_stride(in_per * 4), in_per * 4), rt.DT_F32, buf, rt.DT_U8, in_per, qp(*n.out_qp))
            elif n.op == "conv":
                src = qg.nodes[n.inputs[0]]
                (ph0, ph1), (pw0, pw1) = n.padding
                args = rt.Conv2dArgs(bl, src.out_shape[1], src.out_shape[2], n.stride[0], n.stride[1], 1, 1, ph0, ph1, pw0,
                                     pw1, qp(*src.out_qp), qp(*n.out_qp), n.clamp[0], n.clamp[1], rt.DT_U8)
                if fused_add is not None:
                    add = qg.nodes[fused_add]
                    res_node = add.inputs[0]
                    res = B(res_node)
                    args.residual_dev = res.ptr
                    args.residual_qp = qp(*qg.nodes[res_node].out_qp)
                    args.sum_qp = qp(*add.out_qp)
                    args.sum_clamp_min, args.sum_clamp_max = FULL_CLAMP
                    self.fn._keep.append(res)
                wthru = self.write_through.get(i)
                if wthru is not None:
                    buf = B(wthru[0])
                    args.out_channel_offset, args.out_channel_stride = wthru[1], wthru[2]
                if i in self.fused_dequant:
                    oj = qg.nodes[qg.output_nodes[self.fused_dequant[i]]]
                    per = bl * int(np.prod(oj.out_shape)) * 4
                    buf = self.outputs_f32[self.fused_dequant[i]].view(lane * self._lane_stride(per), per)
                    args.out_dtype, args.dequantize_output = rt.DT_F32, 1
                if i in self.pairs:
                    j = self.pairs[i]
                    sn, sn_in = qg.nodes[j], qg.nodes[j].inputs[0]
                    mid = qg.nodes[sn_in]
                    second = rt.Conv2dArgs(bl, mid.out_shape[1], mid.out_shape[2], 1, 1, 1, 1, 0, 0, 0, 0, qp(*mid.out_qp), qp(*sn.out_qp),
                                           sn.clamp[0], sn.clamp[1], rt.DT_U8)
                    lut2 = self.fused_lut.get(j)
                    d = self.pair_fronts.get(i)
                    if d is not None:
                        dn, dsrc = qg.nodes[d], qg.nodes[qg.nodes[d].inputs[0]]
                        (dh0, dh1), (dw0, dw1) = dn.padding
                        front = rt.Conv2dArgs(bl, dsrc.out_shape[1], dsrc.out_shape[2], dn.stride[0], dn.stride[1], 1, 1, dh0, dh1, dw0, dw1,
                                              qp(*dsrc.out_qp), qp(*dn.out_qp), dn.clamp[0], dn.clamp[1], rt.DT_U8)
                        self.fn.add_qdepthwise_pointwise_pair(B(dn.inputs[0]), self.weights[d], front, self.pair_objects[i], B(sn_in),
                                                              B(lut2 if lut2 is not None else j), args, second)
                        members = [d] + members
                    else:
                        self.fn.add_qpointwise_pair(B(n.inputs[0]), self.pair_objects[i], B(sn_in), B(lut2 if lut2 is not None else j), args, second)
                    if lane == 0:
                        self.op_names.append(("pair:" if d is None else f"pair:{qg.nodes[d].name}>") + n.name + ("+lut" if fused_lut is not None else "")
                                             + ("+add" if fused_add is not None else "") + f">{sn.name}" + ("+lut" if lut2 is not None else ""))
                        self.op_nodes.append(lut2 if lut2 is not None else j)
                        self.op_members.append(members + [j] + ([lut2] if lut2 is not None else []))
                    continue
                if i in self.pool_fronts:
                    g_ = self.pool_fronts[i]
                    gsrc = qg.nodes[qg.nodes[g_].inputs[0]]
                    self.fn.add_qglobal_avgpool_qconv2d(B(qg.nodes[g_].inputs[0]), gsrc.out_shape[1], gsrc.out_shape[2], qp(*gsrc.out_qp),
                                                        self.weights[i], buf, args)
                    if lane == 0:
                        self.op_names.append(f"gap:{qg.nodes[g_].name}>conv:{n.name}" + ("+lut" if fused_lut is not None else ""))
                        self.op_nodes.append(fused_lut if fused_lut is not None else i)
                        self.op_members.append([g_] + members)
                    continue
                self.fn.add_qconv2d(B(n.inputs[0]), self.weights[i], buf, args)
            elif n.op == "add":
                a, b = (qg.nodes[j] for j in n.inputs)
                self.fn.add_qadd(B(n.inputs[0]), qp(*a.out_qp), B(n.inputs[1]), qp(*b.out_qp), buf,
                                 qp(*n.out_qp), bl * cc * hh * ww)
            elif n.op == "lut":
                self.fn.add_lut_u8(B(n.inputs[0]), buf, bl * cc * hh * ww, n.lut)
            elif n.op == "concat":
                srcs = [qg.nodes[j] for j in n.inputs]
                in_place = {jn for conv, (ci_, _o, _s, _t) in self.write_through.items() if ci_ == i
                            for jn in (self.fused_into.get(conv, self.fused_lut.get(conv, conv)),)}
                if len(in_place) == len(n.inputs):
                    continue                                   # every slice is written by its producer
                self.fn.add_qconcat_channels([None if j in in_place else B(j) for j in n.inputs], [s_.out_shape[0] for s_ in srcs],
                                             [qp(*s_.out_qp) for s_ in srcs], buf, qp(*n.out_qp), bl * hh * ww)
            elif n.op == "resize":
                src = qg.nodes[n.inputs[0]]
                self.fn.add_resize_nearest(B(n.inputs[0]), buf, 1, bl, src.out_shape[1], src.out_shape[2], cc, hh, ww,
                                           n.resize_modes[0], n.resize_modes[1])
            elif n.op == "maxpool":
                src = qg.nodes[n.inputs[0]]
                k, st, p = n.pool
                self.fn.add_qmaxpool2d(B(n.inputs[0]), buf, bl, src.out_shape[1], src.out_shape[2], cc, (k, k), (st, st),
                                       ((p, p), (p, p)), qp(*src.out_qp), qp(*n.out_qp))
            elif n.op in ("padc", "s2d"):
                src = qg.nodes[n.inputs[0]]
                sc, sh_, sw_ = src.out_shape
                axes, lns = ([3], [cc]) if n.op == "padc" else ([1, 2, 3], [2, 2, 4])
                if i in self.fused_quant:
                    members = [self.fused_quant[i]] + members    # the operator also computes the input's quantisation
                    self.fn.add_quantize_pack(self.input_f32.view(lane * self._lane_stride(in_per * 4), in_per * 4), buf,
                                              [bl, sh_, sw_, sc], axes, lns, qp(*src.out_qp))
                else:
                    self.fn.add_pack(B(n.inputs[0]), buf, 1, [bl, sh_, sw_, sc], axes, lns)
            elif n.op == "fold2":
                continue
            elif n.op == "gap":
                src = qg.nodes[n.inputs[0]]
                self.fn.add_qglobal_avgpool(B(n.inputs[0]), buf, bl, src.out_shape[1], src.out_shape[2],
                                            src.out_shape[0], qp(*src.out_qp), qp(*n.out_qp))
            else:
                raise ValueError(n.op)
            if lane == 0:
                self.op_names.append(f"{n.op}:{n.name}" + ("+lut" if fused_lut is not None else "") + ("+add" if fused_add is not None else ""))
                self.op_nodes.append(fused_add if fused_add is not None else (fused_lut if fused_lut is not None else i))
                self.op_members.append(members)
        for k, j in enumerate(qg.output_nodes):
            if k in self.fused_dequant.values():
                continue                                       # stored as float32 by the conv that produces it
            node = qg.nodes[j]
            count = bl * int(np.prod(node.out_shape))
            self.fn.add_dequantize(B(j), rt.DT_U8, self.outputs_f32[k].view(lane * self._lane_stride(count * 4), count * 4), rt.DT_F32, count, qp(*node.out_qp))
            if lane == 0:
                self.op_names.append("dequantize:" + node.name)
                self.op_nodes.append(j)
                self.op_members.append([])

    def set_input(self, x_nhwc: np.ndarray):
        x = np.ascontiguousarray(x_nhwc, f32)
        assert x.size == self.in_count, f"expected {self.in_count} input elements, got {x.size}"
        per = self.in_count // self.lanes * 4
        if self._lane_stride(per) == per:
            self.input_f32.upload(x)
        else:
            for lane, part in enumerate(np.split(x.reshape(-1), self.lanes)):
                self.input_f32.view(lane * self._lane_stride(per), per).upload(part)

    def _lane_stride(self, nbytes: int) -> int:
        """Byte distance between the lanes' image ranges of a tensor: the range itself when there is one lane
        or its size keeps every lane 256-byte aligned (the tensor is then one contiguous NHWC array), else the
        size rounded up (the kernels want 16-byte aligned operands)."""
        return nbytes if self.lanes == 1 or nbytes % 256 == 0 else (nbytes + 255) // 256 * 256

    def _download(self, buf, shape, dtype) -> np.ndarray:
        per_shape = (shape[0] // self.lanes,) + tuple(shape[1:])
        per = int(np.prod(per_shape)) * np.dtype(dtype).itemsize
        stride = self._lane_stride(per)
        if stride == per:
            return buf.download(shape, dtype)
        return np.concatenate([buf.view(lane * stride, per).download(per_shape, dtype) for lane in range(self.lanes)])

    def invoke(self):
        self.fn.invoke()

    def output(self, index: int = 0) -> np.ndarray:
        """Dequantised float32 output `index`, NCHW-shaped [batch, C, H, W] (H = W = 1 for classifiers)."""
        c, h, w = self.qg.nodes[self.qg.output_nodes[index]].out_shape
        y = self._download(self.outputs_f32[index], (self.batch, h, w, c), f32)
        return np.ascontiguousarray(y.transpose(0, 3, 1, 2))

    def all_outputs(self) -> List[np.ndarray]:
        return [self.output(i) for i in range(len(self.outputs_f32))]

    def materialized(self, node: int) -> bool:
        """False for a tensor that only exists inside a fused operator (conv + table + residual add)."""
        return node not in self.never_written

    def tensor(self, node: int) -> np.ndarray:
        """u8 output of a node as NCHW (for layer-by-layer parity checks)."""
        if not self.materialized(node):
            raise ValueError(f"node {node} only exists inside a fused operator and is never written")
        c, h, w = self.qg.nodes[node].out_shape
        y = self._download(self.buffers[node], (self.batch, h, w, c), np.uint8)
        return np.ascontiguousarray(y.transpose(0, 3, 1, 2))

    def run(self, x_nhwc: np.ndarray) -> np.ndarray:
        self.set_input(x_nhwc)
        self.invoke()
        self.ctx.sync()
        return self.output()


class HipPipeline:
    """`depth` copies of a HipModel, each on a context of its own (its stream, its activation buffers, its packed
    constants), invoked in turn: batch i + 1 is enqueued while batch i is still running, so the small, latency-bound
    layers at the end of one batch share the device with the bandwidth-bound layers at the start of the next.
    Every batch is computed by one copy from start to finish, so results are the bytes a single HipModel gives.
    This is how a server keeps a device busy with the reference too: one interpreter per request in flight
    (an interpreter is single threaded, src/Native/src/runtime/interpreter.cpp)."""

    def __init__(self, device: int, qg: QuantGraph, batch: int, depth: int = 4, **model_args):
        if depth < 1:
            raise ValueError("depth must be at least 1")
        # HIP multiplexes its streams over at most GPU_MAX_HW_QUEUES (4 unless the environment says otherwise) hardware
        # queues: a new stream opens a new hardware queue until that many exist and joins the least shared one after
        # that, and the kernels of streams that share a hardware queue run one after the other.  Copies beyond the
        # number of hardware queues therefore add nothing, and copies that happen to share a queue while another
        # queue holds only the caller's idle stream halve each other's rate (measured: four copies created right after
        # the caller's own stream give 183 k images/s on MobileNetV2 at batch 64, one per hardware queue 224 k; six or
        # eight hardware queues instead of four give 164-180 k).  So the pool is filled with idle streams first: the
        # copies' streams then land on one hardware queue each.
        self.device = device
        self.hw_queues = rt.fill_queue_pool(device)
        self.contexts = [Context(device) for _ in range(depth)]
        self.models = [HipModel(c, qg, batch, **model_args) for c in self.contexts]
        self.turn = 0

    def set_input(self, x_nhwc: np.ndarray):
        for m in self.models:
            m.set_input(x_nhwc)

    def submit(self) -> "HipModel":
        """Enqueues one batch on the next copy and returns that copy (its output is valid after its context syncs)."""
        m = self.models[self.turn % len(self.models)]
        self.turn += 1
        m.invoke()
        return m

    invoke = submit

    def sync(self):
        for c in self.contexts:
            c.sync()

    def close(self, release_queue_pool: bool = True):
        """Waits for the copies, destroys their contexts and, unless another pipeline still wants it, the pool of idle
        streams that spread the copies over the hardware queues."""
        self.sync()
        self.models = []
        for c in self.contexts:
            c.close()
        self.contexts = []
        if release_queue_pool:
            rt.release_queue_pool(self.device)
