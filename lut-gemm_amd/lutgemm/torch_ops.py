"""PyTorch-ROCm front end of the C ABI: a registered operator and a drop-in linear layer.

  torch.ops.lutgemm.matvec(x, handle)   y[..., n] = x[..., k] @ W  for a packed BCQ weight
  LutLinear                             nn.Module around one packed weight (+ optional bias)

The operator launches on torch's current stream and allocates nothing but its output, so it can
be captured into a HIP graph like any other torch op.  Batches larger than `dense_threshold`
rows go through the dequantised fp16 weight and the library GEMM, the route the reference takes
for every m > 1 (lutGEMM/src/kernels.cu:73-79).  Like the reference, which dequantises into one
grow-only scratch buffer of the process on every such call (lutGEMM/src/cuda/tmpWeight.hpp:28-35,
lutGEMM/src/nQWeight_fp16.cu:93-99), the dense weight is rebuilt per call in a scratch buffer shared
by all layers (one per device and stream), so a layer never holds more than its packed weight;
`keep_dense=True` keeps a private dense copy instead (2 k n bytes) and skips the rebuild.  Up to
the threshold the library streams the packed weight
(one or two rows through the table-lookup kernels, more through the batch kernel, 16 rows per
pass).  The default threshold depends on the weight and on keep_dense (default_dense_threshold):
it is where the two routes met when measured on MI355X.
"""


def default_dense_threshold(weight, keep_dense=False):
    """Rows up to which the packed route beats dequantised weight + library GEMM (measured on MI355X
    at k = n = 12288 and at k = 7168, n = 28672; LutLinear(dense_threshold=...) overrides).

    A pass of the batch kernel over up to 16 rows costs 22 / 24 / 30 / 36 us for one to four planes
    and 41 / 43 / 50 / 57 us for five to eight (k = n = 12288).  The dense route costs the
    dequantisation (75 us up to four planes, 97-130 us for five to eight) plus the GEMM (50-56 us up
    to 32 rows), so by default it only pays from the number of passes on that costs as much:
    80 rows for one or two planes, 64 for three, 48 beyond.  A layer that keeps its dense copy
    (keep_dense) pays the GEMM alone: 32 rows for one or two planes, 16 for three to seven, and
    eight planes leave the packed route from three rows on (57 against 50 us)."""
    q = weight.nb
    if keep_dense:
        return 32 if q <= 2 else 16 if q <= 7 else 2
    return 80 if q <= 2 else 64 if q == 3 else 48


import weakref

import numpy as np
import torch

from . import BCQWeight, LutGemmError, ERR_BAD_SHAPE, MAX_BATCH

_weights = weakref.WeakValueDictionary()  # operator argument (an int) -> BCQWeight
_next_id = [1]
_dense_scratch = {}   # (device index, stream handle) -> grow-only fp16 buffer for dequantised weights


def dense_scratch(halves, device, stream_handle):
    """View of `halves` fp16 elements of the process-wide scratch buffer of (device, stream); the
    buffer only ever grows (the counterpart of the reference's tmpWeight singleton)."""
    key = (device.index, stream_handle)
    buf = _dense_scratch.get(key)
    if buf is None or buf.numel() < halves:
        buf = torch.empty(halves, dtype=torch.float16, device=device)
        _dense_scratch[key] = buf
    return buf[:halves]


def register(weight):
    """Make a BCQWeight addressable by the operator; returns its integer handle."""
    hid = _next_id[0]
    _next_id[0] += 1
    _weights[hid] = weight
    return hid


def _lookup(handle):
    w = _weights.get(int(handle))
    if w is None:
        raise LutGemmError(ERR_BAD_SHAPE, "operator handle %d is not registered (or its weight was freed)" % handle)
    return w


@torch.library.custom_op("lutgemm::matvec", mutates_args=())
def matvec(x: torch.Tensor, handle: int) -> torch.Tensor:
    w = _lookup(handle)
    if not x.is_cuda or x.dtype != torch.float16:
        raise TypeError("lutgemm::matvec needs a float16 tensor on the GPU, got %s on %s" % (x.dtype, x.device))
    if x.shape[-1] != w.kSize:
        raise LutGemmError(ERR_BAD_SHAPE, "last dimension %d != k %d" % (x.shape[-1], w.kSize))
    x2 = x.reshape(-1, w.kSize).contiguous()
    m = x2.shape[0]
    y = torch.empty((m, w.mSize), dtype=torch.float16, device=x.device)
    stream = torch.cuda.current_stream(x.device).cuda_stream
    with torch.cuda.device(x.device):
        for r0 in range(0, m, MAX_BATCH):
            rows = min(MAX_BATCH, m - r0)
            w.matvec(x2[r0:r0 + rows].data_ptr(), y[r0:r0 + rows].data_ptr(), rows, stream)
    return y.reshape(x.shape[:-1] + (w.mSize,))


@matvec.register_fake
def _(x, handle):
    w = _lookup(handle)
    return x.new_empty(x.shape[:-1] + (w.mSize,))


class LutLinear(torch.nn.Module):
    """y = x @ W (+ bias) with W held as a packed BCQ weight on the current device.

    container: dict(bW, alpha, q_bias, k, n, q, num_groups) as quantize.to_container returns.
    """

    def __init__(self, container, bias=None, dense_threshold=None, autotune=False, keep_dense=False):
        super().__init__()
        c = container
        self.device = torch.device("cuda", torch.cuda.current_device())   # the packed weight lives here
        self.keep_dense = keep_dense
        self.weight = BCQWeight(c["bW"], c["alpha"], c["k"], c["n"], c["q"], c["num_groups"], c.get("q_bias"))
        if autotune:
            self.weight.autotune(torch.cuda.current_stream().cuda_stream)
        self.handle = register(self.weight)
        self.in_features, self.out_features = c["k"], c["n"]
        self.dense_threshold = default_dense_threshold(self.weight, keep_dense) if dense_threshold is None else dense_threshold
        self._dense = None
        if bias is not None:
            self.register_buffer("bias", torch.as_tensor(bias).to(torch.float16).to(self.device))
        else:
            self.bias = None

    @classmethod
    def from_file(cls, path, bias=None, **kw):
        self = cls.__new__(cls)
        torch.nn.Module.__init__(self)
        self.device = torch.device("cuda", torch.cuda.current_device())
        self.keep_dense = kw.get("keep_dense", False)
        self.weight = BCQWeight.load(path)
        if kw.get("autotune", False):
            self.weight.autotune(torch.cuda.current_stream().cuda_stream)
        self.handle = register(self.weight)
        self.in_features, self.out_features = self.weight.kSize, self.weight.mSize
        dt = kw.get("dense_threshold")
        self.dense_threshold = default_dense_threshold(self.weight, self.keep_dense) if dt is None else dt
        self._dense = None
        if bias is not None:
            self.register_buffer("bias", torch.as_tensor(bias).to(torch.float16).to(self.device))
        else:
            self.bias = None
        return self

    @classmethod
    def from_linear(cls, linear, qbits, group_size=128, method="rtn", rounds=15, **kw):
        """Quantise a torch.nn.Linear (weight [out, in]) and pack it."""
        from . import quantize
        c, _ = quantize.quantize_linear(linear.weight.detach().float(), qbits, group_size, method, rounds)
        b = None if linear.bias is None else linear.bias.detach()
        return cls(c, bias=b, **kw)

    def dense_weight(self):
        """Dequantised fp16 weight on the layer's device as W^T [n][k], the orientation the
        dequantise kernel writes in 1 KiB runs.  Rebuilt on torch's current stream into the shared
        scratch buffer of that stream on every call (valid until the next layer's call on the
        stream); with keep_dense it is built once and kept by the layer."""
        if self._dense is not None:
            return self._dense
        stream = torch.cuda.current_stream(self.device).cuda_stream
        if self.keep_dense:
            Wt = torch.empty((self.out_features, self.in_features), dtype=torch.float16, device=self.device)
        else:
            Wt = dense_scratch(self.out_features * self.in_features, self.device, stream).view(self.out_features, self.in_features)
        with torch.cuda.device(self.device):
            self.weight.dequantize(Wt.data_ptr(), True, stream)
        if self.keep_dense:
            self._dense = Wt
        return Wt

    def forward(self, x):
        rows = x.numel() // x.shape[-1]
        x = x.to(torch.float16)
        if rows > self.dense_threshold:
            y = torch.nn.functional.linear(x, self.dense_weight())
        else:
            y = torch.ops.lutgemm.matvec(x, self.handle)
        return y if self.bias is None else y + self.bias


def container_from_numpy(bW, alpha, k, n, q, num_groups, q_bias=None):
    return dict(bW=np.asarray(bW), alpha=np.asarray(alpha), q_bias=q_bias, k=k, n=n, q=q, num_groups=num_groups)
