"""Weight quantisers that end in a BCQ container for the LUT matvec.

Counterparts of the reference's Python examples, written for torch tensors on any device (the
input's device is used; nothing here requires a GPU):

  rtn_quantize      round-to-nearest uniform quantisation per group (examples/utils.py:52-124,
                    examples/rtn_parameter.py:25-54, min/max variant)
  rtn_to_bcq        uniform codes written as binary-coding planes plus an offset
                    (examples/rtn_parameter.py:77-96)
  quantize          greedy binary-coding quantisation refined by alternating least squares, with
                    the weighting factors (exponent, clipping, pruning), the transposed grouping
                    and both sign-assignment rules of examples/bcq.py:22-206
  bcq_quantize      the same without weighting, three return values
  Packer            eight -1/+1 entries per byte (examples/utils.py:149-183)
  RTNParameter, BCQParameter   compress / decompress / convert_bcq_format with the argument names
                    of examples/rtn_parameter.py:25-96 and examples/bcq_parameter.py:22-61
  quantize_model    walk a torch model and quantise its projection layers
                    (examples/quant_model_rtn.py:67-98, examples/quant_model_bcq.py:66-84)
  dequantize_bcq    sum_b alpha_b * binary_b (+ offset) (examples/bcq_parameter.py:36-61)
  to_container      out-major example layout -> the [k/32][q][n] / [G][q][n] / [G][n] arrays that
                    nQWeight_fp16::parsing takes (lutGEMM/src/nQWeight_fp16.cu:60-91)

Layouts follow the examples with in_ch_wise=False: a linear weight w is [out, in]; groups run
along `in`; binary is [out, in/g, g, q] with entries -1/+1, alpha [out, in/g, q], offset
[out, in/g, 1].  The matvec computes y = x @ w.T, i.e. k = in and n = out.
"""
import numpy as np
import torch


def _groups(w, group_size):
    out_ch, in_ch = w.shape
    g = in_ch if group_size is None or group_size <= 0 else group_size
    if in_ch % g != 0:
        raise ValueError("in_features %d is not a multiple of group_size %d" % (in_ch, g))
    return out_ch, in_ch, g


def _uniform(x, scale, zero, maxq):
    return scale * (torch.clamp(torch.round(x / scale) + zero, 0, maxq) - zero)


@torch.no_grad()
def rtn_quantize(w, qbits, group_size=-1, sym=False, mse=False, norm=2.4, grid=100, maxshrink=0.8,
                 perchannel=True):
    """Uniform quantisation with one (scale, zero) per group of `group_size` input channels.

    Returns (scale [out, G, 1], zero [out, G, 1], codes int32 [out, G, g]) with
    w ~= scale * (codes - zero), codes in 0 .. 2^qbits - 1.  The range of a group always includes
    zero; sym=True makes it symmetric about zero.  mse=True shrinks the range of each group in
    `grid` steps down to (1 - maxshrink) of it and keeps the (scale, zero) with the smallest
    sum |error|^norm (the search of examples/utils.py:91-110).  perchannel=False shares one
    (scale, zero) over the whole tensor (examples/utils.py:69-70, 111-117).
    """
    out_ch, in_ch, g = _groups(w, group_size)
    maxq = float(2 ** qbits - 1)
    x = w.detach().to(torch.float32).reshape(-1, g)
    rows = x.shape[0]
    if not perchannel:
        x = x.reshape(1, -1)
    zeros = torch.zeros(x.shape[0], device=x.device)
    xmin = torch.minimum(x.min(dim=1).values, zeros)
    xmax = torch.maximum(x.max(dim=1).values, zeros)
    if sym:
        xmax = torch.maximum(xmin.abs(), xmax)
        xmin = torch.where(xmin < 0, -xmax, xmin)
    flat = (xmin == 0) & (xmax == 0)
    xmin = torch.where(flat, torch.full_like(xmin, -1.0), xmin)
    xmax = torch.where(flat, torch.full_like(xmax, 1.0), xmax)
    scale = (xmax - xmin) / maxq
    zero = torch.full_like(scale, (maxq + 1) / 2) if sym else torch.round(-xmin / scale)
    if mse:
        best = torch.full_like(scale, float("inf"))
        full_zero = zero.clone()
        for i in range(int(maxshrink * grid)):
            p = 1.0 - i / grid
            scale1 = p * (xmax - xmin) / maxq
            zero1 = full_zero if sym else torch.round(-(p * xmin) / scale1)
            err = (_uniform(x, scale1[:, None], zero1[:, None], maxq) - x).abs().pow(norm).sum(dim=1)
            better = err < best
            best = torch.where(better, err, best)
            scale = torch.where(better, scale1, scale)
            zero = torch.where(better, zero1, zero)
    codes = torch.clamp(torch.round(x / scale[:, None]) + zero[:, None], 0, maxq).to(torch.int32)
    if not perchannel:
        scale, zero = scale.repeat(rows), zero.repeat(rows)
    G = in_ch // g
    return scale.reshape(out_ch, G, 1), zero.reshape(out_ch, G, 1), codes.reshape(out_ch, G, g)


@torch.no_grad()
def rtn_dequantize(scale, zero, codes):
    out_ch = codes.shape[0]
    return (scale * (codes.to(scale.dtype) - zero)).reshape(out_ch, -1)


@torch.no_grad()
def rtn_to_bcq(scale, zero, codes, qbits):
    """scale * (c - zero) with c = sum_i 2^i bit_i, rewritten with signs s_i = 2 bit_i - 1:
    alpha_i = scale * 2^i / 2 (least significant plane first), offset = sum_i alpha_i - scale*zero.
    Returns (alpha [out, G, q], binary [out, G, g, q] of -1/+1, offset [out, G, 1])."""
    pow2 = torch.tensor([2.0 ** i for i in range(qbits)], dtype=scale.dtype, device=scale.device)
    alpha = (scale / 2.0) * pow2  # [out, G, q]
    offset = alpha.sum(-1, keepdim=True) - scale * zero
    shifts = torch.arange(qbits, device=codes.device, dtype=torch.int32)
    bits = (codes.to(torch.int32)[..., None] >> shifts) & 1
    binary = bits.to(scale.dtype) * 2.0 - 1.0
    return alpha, binary, offset


def _sign_pm1(r):
    # zeros count as +1: every weight needs a sign bit in the packed planes
    return torch.where(r >= 0, torch.ones_like(r), -torch.ones_like(r))


def _greedy(x, qbits, wf=None):
    """b_i = sign(residual), alpha_i = (weighted) mean |residual|, plane after plane."""
    B = torch.empty(x.shape + (qbits,), dtype=x.dtype, device=x.device)
    A = torch.empty((x.shape[0], qbits), dtype=x.dtype, device=x.device)
    r = x.clone()
    for i in range(qbits):
        b = _sign_pm1(r)
        if wf is None:
            a = r.abs().mean(dim=1, keepdim=True)
        else:
            a = torch.nan_to_num((r.abs() * wf).sum(dim=1, keepdim=True) / wf.sum(dim=1, keepdim=True), nan=0.0)
        r -= b * a
        B[:, :, i] = b
        A[:, i] = a[:, 0]
    return B, A


def _sign_patterns(qbits, dtype, device):
    idx = torch.arange(2 ** qbits, device=device)
    bits = (idx[:, None] >> torch.arange(qbits, device=device)) & 1
    return bits.to(dtype) * 2.0 - 1.0  # [2^q, q]


def _refine(x, B, A, wf=None, use_bst=True):
    """One alternating round: scales by (weighted) least squares for the current signs, made
    non-negative and sorted (a relabelling of the planes); then the signs again, either every
    weight to its nearest level (use_bst) or greedily plane after plane.  Weights whose factor is
    zero (pruned) get the code 0 in every plane under use_bst, as in examples/bcq.py:151-152."""
    q = A.shape[1]
    Bw = B if wf is None else B * wf[..., None]
    BtB = torch.einsum("rgi,rgj->rij", Bw, B)
    Btw = torch.einsum("rgi,rg->ri", Bw, x)
    eye = torch.eye(q, dtype=x.dtype, device=x.device)
    A_new = torch.linalg.solve(BtB + 1e-6 * eye, Btw[..., None])[..., 0]
    A_new = A_new.abs().sort(dim=1, descending=True).values
    if not use_bst:
        r = x.clone()
        B_new = torch.empty_like(B)
        for i in range(q):
            B_new[:, :, i] = _sign_pm1(r)
            r -= B_new[:, :, i] * A_new[:, i:i + 1]
        return B_new, A_new
    pats = _sign_patterns(q, x.dtype, x.device)           # [L, q]
    levels = A_new @ pats.t()                              # [rows, L]
    lv, order = levels.sort(dim=1)
    mids = ((lv[:, 1:] + lv[:, :-1]) / 2).contiguous()
    # a weight exactly between two levels goes to the upper one, as the `w < mid` test of
    # examples/bcq.py:177-181 decides
    pos = torch.searchsorted(mids, x.contiguous(), right=True)   # index into the sorted levels
    which = torch.gather(order, 1, pos)                    # pattern index per weight
    B_new = pats[which]                                    # [rows, g, q]
    if wf is not None:
        B_new = B_new * (wf != 0)[..., None]
    return B_new, A_new


def _weight_factors(x, exponent, clipping, pruning):
    """Per-weight importance of the weighted variant (examples/bcq.py:52-76): |w| / max|w|,
    saturated at the `clipping` quantile, raised to `exponent`; the `pruning` fraction of smallest
    |w| gets factor 0 and is set to zero in x (in place).  None when every factor is 1."""
    if not (exponent > 0.0 or clipping < 1.0 or pruning > 0.0):
        return None
    w_abs = x.abs()
    ws = w_abs.reshape(-1).sort().values
    wf = torch.ones_like(x)
    if pruning > 0.0:
        wf = wf * (x != 0.0)
    if exponent > 0.0 or clipping < 1.0:
        wf = w_abs / w_abs.max()
    if clipping < 1.0:
        c_th = ws[min(int(ws.numel() * clipping), ws.numel() - 1)]
        wf = torch.clamp(wf * w_abs.max() / c_th, max=1.0)
    if exponent > 0.0:
        wf = wf ** exponent
    if pruning > 0.0:
        p_th = ws[min(int(ws.numel() * pruning), ws.numel() - 1)]
        low = w_abs <= p_th
        wf = torch.where(low, torch.zeros_like(wf), wf)
        x[low] = 0.0
    return wf


@torch.no_grad()
def quantize(w, qbits, rounds=15, group_size=-1, transpose=False, exponent=0.0, clipping=1.0, pruning=0.0,
             use_bst=True):
    """Binary-coding quantisation w ~= sum_i alpha_i * b_i per group, argument for argument the
    `quantize` of examples/bcq.py:22-96: greedy start, then `rounds` alternating refinements
    (rounds=0 is the plain greedy result).  transpose=True groups along the first dimension of w
    (binary [in, out/g, g, q]).  Computed on the device w lives on.

    Returns (w_hat shaped like w, binary [d0, G, g, q], alpha [d0, G, q], kept [d0*G, g] bool);
    alpha is non-negative and, after any refinement, sorted in descending order; `kept` is False
    for pruned weights, whose binary entries are 0 (such a result has no packed form).
    """
    x2 = w.detach().to(torch.float32)
    if transpose:
        if x2.dim() != 2:
            raise ValueError("transpose needs a 2-d weight, got shape %s" % (tuple(w.shape),))
        x2 = x2.t()
    d0, d1, g = _groups(x2, group_size)
    x = x2.reshape(-1, g).clone()
    wf = _weight_factors(x, exponent, clipping, pruning)
    B, A = _greedy(x, qbits, wf)
    if qbits > 1:
        for _ in range(rounds):
            B, A = _refine(x, B, A, wf, use_bst)
    if wf is not None:
        # pruned weights (factor 0, value set to 0) keep the code 0 in every plane on every route
        # (the reference's r.sign() of a zero residual, examples/bcq.py:106), not only under use_bst
        B = B * (wf != 0)[..., None]
    w_hat = torch.einsum("rgq,rq->rg", B, A).reshape(d0, d1)
    if transpose:
        w_hat = w_hat.t().contiguous()
    kept = torch.ones_like(x, dtype=torch.bool) if wf is None else (wf != 0)
    G = d1 // g
    return w_hat, B.reshape(d0, G, g, qbits), A.reshape(d0, G, qbits), kept


@torch.no_grad()
def bcq_quantize(w, qbits, rounds=15, group_size=-1):
    """Unweighted `quantize` with groups along the input channels.

    Returns (w_hat [out, in], binary [out, G, g, q] of -1/+1, alpha [out, G, q]).
    """
    w_hat, binary, alpha, _ = quantize(w, qbits, rounds, group_size)
    return w_hat, binary, alpha


@torch.no_grad()
def dequantize_bcq(binary, alpha, offset=None, in_ch_wise=False):
    """[out, in] weight from binary [d0, G, g, q], alpha [d0, G, q], offset [d0, G, 1]; with
    in_ch_wise the first dimension is the input channel and the groups run along the outputs."""
    w = torch.einsum("oigb,oib->oig", binary.to(alpha.dtype), alpha)
    if offset is not None:
        w = w + offset
    w = w.reshape(binary.shape[0], -1)
    return w.t() if in_ch_wise else w


@torch.no_grad()
def to_container(binary, alpha, offset=None):
    """Example layout -> container arrays (numpy): bW uint32 [k/32][q][n] with bit t of word w
    = 1 iff the sign of input channel 32 w + t is +1, alpha float32 [G][q][n], q_bias float32
    [G][n] or None.  k = in_features must be a multiple of 32."""
    out_ch, G, g, q = binary.shape
    k = G * g
    if k % 32 != 0:
        raise ValueError("in_features %d is not a multiple of 32" % k)
    if bool((binary == 0).any()):
        raise ValueError("binary holds zeros (pruned weights): a sign plane stores -1/+1 only")
    bits = (binary.reshape(out_ch, k, q) > 0).permute(2, 0, 1).contiguous().cpu().numpy()      # [q][n][k]
    packed = np.packbits(bits, axis=-1, bitorder="little")                                      # [q][n][k/8]
    bW = np.ascontiguousarray(packed).view("<u4").transpose(2, 0, 1)                             # [k/32][q][n]
    alpha_c = alpha.permute(1, 2, 0).contiguous().to(torch.float32).cpu().numpy()
    q_bias = None
    if offset is not None:
        q_bias = offset.reshape(out_ch, G).t().contiguous().to(torch.float32).cpu().numpy()
    return dict(bW=np.ascontiguousarray(bW), alpha=alpha_c, q_bias=q_bias, k=k, n=out_ch, q=q, num_groups=G, g=g)


class Packer:
    """Eight -1/+1 entries per byte, the packing of examples/utils.py:149-183: the flattened
    tensor of N entries (N a multiple of 8) is cut into eight runs of N/8; bit i of byte j is 1 iff
    entry i*N/8 + j is +1."""

    def pack(self, b):
        shape = b.shape
        bits = ((b.reshape(8, -1) + 1) / 2).to(torch.uint8)
        weights = torch.tensor([1, 2, 4, 8, 16, 32, 64, 128], dtype=torch.uint8, device=b.device).reshape(8, 1)
        return (bits * weights).sum(0).to(torch.uint8), shape

    def unpack(self, pb, shape, dtype=torch.float16):
        shifts = torch.arange(8, device=pb.device, dtype=torch.uint8).reshape(8, 1)
        bits = (pb.reshape(1, -1) >> shifts) & 1
        return (bits.to(dtype) * 2 - 1).reshape(shape)


PACKER = Packer()


class CompressionParameter:
    """Holder of one weight tensor in `.data` (the reference derives it from nn.Parameter,
    examples/utils.py:185-190; nothing here needs autograd)."""

    def __init__(self, data):
        self.data = data


class RTNParameter(CompressionParameter):
    """examples/rtn_parameter.py:25-96 with its argument names."""

    def compress(self, in_ch_wise=False, group_size=-1, **kwargs):
        """kwargs: qbits, perchannel, sym, mse, norm, grid, maxshrink.  Returns (scale, zero,
        codes, codes.shape) with codes [d0, G, g]; d0 = out (groups along in), or in when in_ch_wise."""
        kwargs.setdefault("sym", True)          # the defaults of examples/utils.py:36-38
        kwargs.setdefault("perchannel", False)
        data = self.data.t() if in_ch_wise else self.data
        scale, zero, codes = rtn_quantize(data, group_size=group_size, **kwargs)
        return scale, zero, codes, codes.shape

    def decompress(self, scale, zero, quant_data, quant_data_shape, in_ch_wise=False):
        w = rtn_dequantize(scale, zero, quant_data)
        self.data = w.t() if in_ch_wise else w

    def convert_bcq_format(self, scale, zero, quant_data, qbits, do_packing=False, in_ch_wise=False):
        alpha, binary, offset = rtn_to_bcq(scale, zero, quant_data, qbits)
        binary_shape = binary.shape
        if do_packing:
            binary, binary_shape = PACKER.pack(binary)
        return alpha, binary, binary_shape, offset


class BCQParameter(CompressionParameter):
    """examples/bcq_parameter.py:22-61 with its argument names."""

    def compress(self, do_packing=False, in_ch_wise=False, **kwargs):
        """kwargs: qbits, rounds, group_size, exponent, clipping, pruning, use_bst."""
        _, binary, alpha, _ = quantize(self.data, transpose=in_ch_wise, **kwargs)
        binary_shape = binary.shape
        if do_packing:
            binary, binary_shape = PACKER.pack(binary)
        return alpha, binary, binary_shape

    def decompress(self, alpha, binary, binary_shape, offset=None, do_packing=False, in_ch_wise=False):
        if do_packing:
            binary = PACKER.unpack(binary, binary_shape, dtype=alpha.dtype)
        self.data = dequantize_bcq(binary, alpha, offset, in_ch_wise)


def quantize_linear(weight, qbits, group_size=128, method="rtn", rounds=15):
    """[out, in] weight -> (container dict for BCQWeight / pack_file, dequantised weight [out, in])."""
    if method == "rtn":
        scale, zero, codes = rtn_quantize(weight, qbits, group_size)
        alpha, binary, offset = rtn_to_bcq(scale, zero, codes, qbits)
        return to_container(binary, alpha, offset), rtn_dequantize(scale, zero, codes)
    if method == "bcq":
        w_hat, binary, alpha = bcq_quantize(weight, qbits, rounds, group_size)
        return to_container(binary, alpha, None), w_hat
    raise ValueError("method must be 'rtn' or 'bcq'")


# projection layers of an OPT decoder block, the ones the reference's model walkers convert
DEFAULT_LAYERS = ("q_proj", "k_proj", "v_proj", "out_proj", "fc1", "fc2")


def quantize_model(model, qbits=4, group_size=128, method="rtn", rounds=15, layers=DEFAULT_LAYERS,
                   to_device=True, **layer_kw):
    """Quantise every torch.nn.Linear child whose name contains one of `layers`, walking the
    module tree like examples/quant_model_rtn.py:67-98 and examples/quant_model_bcq.py:66-84.

    to_device=True replaces each such layer by a LutLinear on the current GPU (bias kept) and
    returns the model; to_device=False leaves the model alone and returns {qualified name:
    container dict}, e.g. to write files with pack_file.
    """
    found = {}

    def walk(module, prefix):
        for name, child in list(module.named_children()):
            full = prefix + name
            walk(child, full + ".")
            if isinstance(child, torch.nn.Linear) and any(x in name for x in layers):
                if to_device:
                    from .torch_ops import LutLinear
                    setattr(module, name, LutLinear.from_linear(child, qbits, group_size, method, rounds, **layer_kw))
                    found[full] = None
                else:
                    found[full] = quantize_linear(child.weight.detach().float(), qbits, group_size, method, rounds)[0]

    walk(model, "")
    if not found:
        raise ValueError("no torch.nn.Linear child matches %s" % (tuple(layers),))
    return model if to_device else found


def load_packed_model(model, directory, layers=DEFAULT_LAYERS, **layer_kw):
    """Replace every torch.nn.Linear child whose name contains one of `layers` and for which
    <directory>/<qualified name>.lutw exists (as `python -m lutgemm.quant_model` writes them) by
    a LutLinear read from that file on the current GPU; the layer keeps its bias.  Returns the
    list of replaced layer names; raises if no file matches."""
    import os

    from .torch_ops import LutLinear
    done = []

    def walk(module, prefix):
        for name, child in list(module.named_children()):
            full = prefix + name
            walk(child, full + ".")
            path = os.path.join(directory, full + ".lutw")
            if isinstance(child, torch.nn.Linear) and any(x in name for x in layers) and os.path.exists(path):
                bias = None if child.bias is None else child.bias.detach()
                lut = LutLinear.from_file(path, bias=bias, **layer_kw)
                if (lut.in_features, lut.out_features) != (child.in_features, child.out_features):
                    raise ValueError("%s holds a %dx%d weight, layer %s is %dx%d" % (
                        path, lut.in_features, lut.out_features, full, child.in_features, child.out_features))
                setattr(module, name, lut)
                done.append(full)

    walk(model, "")
    if not done:
        raise ValueError("no packed-weight file in %s matches a layer of the model" % directory)
    return done
