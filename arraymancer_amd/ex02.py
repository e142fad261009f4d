"""The forward pass of the reference's example 2 (examples/ex02_handwritten_digits_recognition.nim:36-46),
composed from the device operators of this package:

    x.cv1.relu.mp1.cv2.relu.mp2.fl.hidden.relu.classifier
    cv1 = Conv2D(1 -> 20, 5x5)   mp1 = MaxPool2D(2x2, stride 2)   cv2 = Conv2D(20 -> 50, 5x5)   mp2 = MaxPool2D(2x2, stride 2)
    fl = Flatten                 hidden = Linear(800 -> 500)      classifier = Linear(500 -> 10)

Each convolution is the reference's im2col + GEMM (nn_primitives/fallback/conv.nim:81-106) as ONE batched GEMM
whose B loader gathers the column matrix from the images, with the bias and the ReLU that follows it fused into
the epilogue; each dense layer is one GEMM with fused bias (+ ReLU) (nn_primitives/nnp_linear.nim:20-29); max
pooling is nn_primitives/nnp_maxpooling.nim:19-66. Every buffer is allocated once in the constructor, so that
`forward` issues six kernel launches and nothing else and can be recorded into a HIP graph.
"""
from __future__ import annotations

import ctypes

import numpy as np

from . import _lib
from ._lib import check
from .tensor_hip import Graph, HipTensor, conv2d_into, empty, gemm, toHip


class DemoNet:
    def __init__(self, batch: int, params: dict, dtype=np.float32, hw=(28, 28)):
        """params: cv1_w [20,1,5,5], cv1_b [20], cv2_w [50,20,5,5], cv2_b [50], hidden_w [500,800], hidden_b [1,500],
        classifier_w [10,500], classifier_b [1,10] as host arrays."""
        self.batch, self.dtype = batch, np.dtype(dtype)
        self.p = {k: toHip(np.asarray(v, dtype=dtype)) for k, v in params.items()}
        H, W = hw
        c1, c2 = self.p["cv1_w"].shape[0], self.p["cv2_w"].shape[0]
        k1, k2 = self.p["cv1_w"].shape[2], self.p["cv2_w"].shape[2]
        h1, w1 = H - k1 + 1, W - k1 + 1                 # 24 x 24
        hp1, wp1 = h1 // 2, w1 // 2                     # 12 x 12
        h2, w2 = hp1 - k2 + 1, wp1 - k2 + 1             # 8 x 8
        hp2, wp2 = h2 // 2, w2 // 2                     # 4 x 4
        e = lambda *shape: empty(shape, dtype)
        self.a1 = e(batch, c1, h1, w1)
        self.pool1, self.idx1 = e(batch, c1, hp1, wp1), empty((batch * c1 * hp1 * wp1,), np.int64)
        self.a2 = e(batch, c2, h2, w2)
        self.pool2, self.idx2 = e(batch, c2, hp2, wp2), empty((batch * c2 * hp2 * wp2,), np.int64)
        self.hidden, self.logits = e(batch, self.p["hidden_w"].shape[0]), e(batch, self.p["classifier_w"].shape[0])
        if c2 * hp2 * wp2 != self.p["hidden_w"].shape[1]:
            raise ValueError("hidden layer width does not match the flattened pooling output")

    def _maxpool(self, x: HipTensor, out: HipTensor, idx: HipTensor):
        N, C, H, W = x.shape
        check(getattr(_lib.load(), f"am_hip_maxpool2d_{x.sfx}")(
            N, C, H, W, 2, 2, 0, 0, 2, 2, ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(out.data_ptr()),
            ctypes.c_void_p(idx.data_ptr())))

    def forward(self, x: HipTensor) -> HipTensor:
        """x: [batch, 1, 28, 28] on the device. Returns the [batch, 10] logits (a buffer of this object)."""
        p = self.p
        conv2d_into(self.a1, x, p["cv1_w"], p["cv1_b"], relu=True)
        self._maxpool(self.a1, self.pool1, self.idx1)
        conv2d_into(self.a2, self.pool1, p["cv2_w"], p["cv2_b"], relu=True)
        self._maxpool(self.a2, self.pool2, self.idx2)
        flat = self.pool2.reshape(self.batch, self.pool2.size // self.batch)          # Flatten: metadata only
        gemm(1, flat, p["hidden_w"].transpose(), 0, self.hidden, epilogue="bias_relu", bias=p["hidden_b"])
        gemm(1, self.hidden, p["classifier_w"].transpose(), 0, self.logits, epilogue="bias", bias=p["classifier_b"])
        return self.logits

    def capture(self, x: HipTensor) -> Graph:
        """Records one forward pass over `x` into a HIP graph (run one eager pass first: the GEMM workspace must
        exist before a capture)."""
        self.forward(x)
        with Graph() as g:
            self.forward(x)
        return g.keep(x)


def random_params(rng, dtype=np.float32, scale=0.1) -> dict:
    g = lambda *shape: rng.normal(0, scale, shape).astype(dtype)
    return dict(cv1_w=g(20, 1, 5, 5), cv1_b=g(20), cv2_w=g(50, 20, 5, 5), cv2_b=g(50),
                hidden_w=g(500, 800), hidden_b=g(1, 500), classifier_w=g(10, 500), classifier_b=g(1, 10))
