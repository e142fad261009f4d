"""The network of the reference's example 2 (examples/ex02_handwritten_digits_recognition.nim:36-46), its forward pass
and one step of its learning loop (:58-72), composed from the device operators of this package:

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
from .tensor_hip import (Graph, HipTensor, _unary_into, conv2d_backward, conv2d_into, empty, gemm, linear_backward,
                         maxpool2d_backward, relu_backward, sparse_softmax_cross_entropy,
                         sparse_softmax_cross_entropy_backward, sgd_update, toHip)


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

    def loss_and_gradients(self, x: HipTensor, labels: HipTensor, with_loss: bool = True):
        """One training pass of the example's learning loop (examples/ex02_handwritten_digits_recognition.nim:58-72)
        without the update: forward, `sparse_softmax_cross_entropy` against the int64 `labels` [batch], and what
        `loss.backprop()` walks through, composed from the backward primitives in the order of the forward pass
        reversed (nnp_softmax_cross_entropy.nim:217-256, nnp_linear.nim:39-66, nnp_activation.nim:65-70,
        nnp_maxpooling.nim:68-83, nnp_convolution.nim:65-107). Returns (loss, gradients by parameter name)."""
        p, n = self.p, self.batch
        logits = self.forward(x)
        loss = sparse_softmax_cross_entropy(logits, labels) if with_loss else None
        d_logits = sparse_softmax_cross_entropy_backward(1, logits, labels)
        flat = self.pool2.reshape(n, self.pool2.size // n)
        d_hidden, g_cw, g_cb = linear_backward(self.hidden, p["classifier_w"], d_logits)
        d_hidden = relu_backward(d_hidden, self.hidden)
        d_flat, g_hw, g_hb = linear_backward(flat, p["hidden_w"], d_hidden)
        pool = dict(kernel=(2, 2), padding=(0, 0), stride=(2, 2))
        d_a2 = maxpool2d_backward(self.a2.shape, self.idx2, d_flat.reshape(*self.pool2.shape), **pool)
        d_a2 = relu_backward(d_a2, self.a2)
        d_pool1, g_k2, g_b2 = conv2d_backward(self.pool1, p["cv2_w"], p["cv2_b"], (0, 0), (1, 1), d_a2)
        d_a1 = maxpool2d_backward(self.a1.shape, self.idx1, d_pool1, **pool)
        d_a1 = relu_backward(d_a1, self.a1)
        _, g_k1, g_b1 = conv2d_backward(x, p["cv1_w"], p["cv1_b"], (0, 0), (1, 1), d_a1, need_input_grad=False)
        return loss, dict(cv1_w=g_k1, cv1_b=g_b1, cv2_w=g_k2, cv2_b=g_b2, hidden_w=g_hw, hidden_b=g_hb,
                          classifier_w=g_cw, classifier_b=g_cb)

    def sgd_update(self, gradients: dict, learning_rate: float):
        """The SGD optimizer's update (src/arraymancer/nn/optimizers/optimizers.nim:35-51: x - lr * y over every
        parameter) as ONE launch over all eight parameters."""
        names = list(gradients)
        sgd_update([self.p[k] for k in names], [gradients[k].reshape(*self.p[k].shape) for k in names], learning_rate)

    def gradients(self, x: HipTensor, labels: HipTensor) -> dict:
        """`loss_and_gradients` without the loss: device work only, so that it can be recorded into a graph."""
        return self.loss_and_gradients(x, labels, with_loss=False)[1]

    def capture_train_step(self, x: HipTensor, labels: HipTensor, learning_rate: float = 0.01) -> Graph:
        """One whole learning step (forward, backward, update; the loss is not read back) as ONE graph over the
        buffers `x` and `labels`: refill them and launch. About forty kernels per replay and no host work in between."""
        def step():
            self.sgd_update(self.gradients(x, labels), learning_rate)
        before = {k: v.clone() for k, v in self.p.items()}      # the rehearsal and the capture are not steps of the training
        g = Graph.record(step)
        for k, v in before.items():
            _unary_into("copy", self.p[k], v)
        return g.keep(x, labels)

    def train_step(self, x: HipTensor, labels: HipTensor, learning_rate: float = 0.01):
        loss, gradients = self.loss_and_gradients(x, labels)
        self.sgd_update(gradients, learning_rate)
        return loss

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
