"""Weight quantisers that end in a BCQ container for the LUT matvec.

Counterparts of the reference's Python examples, written for torch tensors on any device (the
input's device is used; nothing here requires a GPU):

  rtn_quantize      round-to-nearest uniform quantisation per group (examples/utils.py:52-124,
                    examples/rtn_parameter.py:25-54, min/max variant)
  rtn_to_bcq        uniform codes written as binary-coding planes plus an offset
                    (examples/rtn_parameter.py:77-96)
  bcq_quantize      greedy binary-coding quantisation refined by alternating least squares
                    (examples/bcq.py:22-206, unweighted case)
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
def rtn_quantize(w, qbits, group_size=-1, sym=False, mse=False, norm=2.4, grid=100, maxshrink=0.8):
    """Uniform quantisation with one (scale, zero) per group of `group_size` input channels.

    Returns (scale [out, G, 1], zero [out, G, 1], codes int32 [out, G, g]) with
    w ~= scale * (codes - zero), codes in 0 .. 2^qbits - 1.  The range of a group always includes
    zero; sym=True makes it symmetric about zero.  mse=True shrinks the range of each group in
    `grid` steps down to (1 - maxshrink) of it and keeps the (scale, zero) with the smallest
    sum |error|^norm (the search of examples/utils.py:91-110).
    """
    out_ch, in_ch, g = _groups(w, group_size)
    maxq = float(2 ** qbits - 1)
    x = w.detach().to(torch.float32).reshape(-1, g)
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


def _greedy(x, qbits):
    """b_i = sign(residual), alpha_i = mean |residual|, plane after plane."""
    B = torch.empty(x.shape + (qbits,), dtype=x.dtype, device=x.device)
    A = torch.empty((x.shape[0], qbits), dtype=x.dtype, device=x.device)
    r = x.clone()
    for i in range(qbits):
        b = _sign_pm1(r)
        a = r.abs().mean(dim=1, keepdim=True)
        r -= b * a
        B[:, :, i] = b
        A[:, i] = a[:, 0]
    return B, A


def _sign_patterns(qbits, dtype, device):
    idx = torch.arange(2 ** qbits, device=device)
    bits = (idx[:, None] >> torch.arange(qbits, device=device)) & 1
    return bits.to(dtype) * 2.0 - 1.0  # [2^q, q]


def _refine(x, B, A):
    """One alternating round: scales by least squares for the current signs, made non-negative
    and sorted (a relabelling of the planes), then every weight moves to its nearest level."""
    q = A.shape[1]
    BtB = torch.einsum("rgi,rgj->rij", B, B)
    Btw = torch.einsum("rgi,rg->ri", B, x)
    eye = torch.eye(q, dtype=x.dtype, device=x.device)
    A_new = torch.linalg.solve(BtB + 1e-6 * eye, Btw[..., None])[..., 0]
    A_new = A_new.abs().sort(dim=1, descending=True).values
    pats = _sign_patterns(q, x.dtype, x.device)           # [L, q]
    levels = A_new @ pats.t()                              # [rows, L]
    lv, order = levels.sort(dim=1)
    mids = ((lv[:, 1:] + lv[:, :-1]) / 2).contiguous()
    pos = torch.searchsorted(mids, x.contiguous())         # index into the sorted levels
    which = torch.gather(order, 1, pos)                    # pattern index per weight
    B_new = pats[which]                                    # [rows, g, q]
    return B_new, A_new


@torch.no_grad()
def bcq_quantize(w, qbits, rounds=15, group_size=-1):
    """Binary-coding quantisation w ~= sum_i alpha_i * b_i per group: greedy start, then `rounds`
    alternating refinements (rounds=0 is the plain greedy result).

    Returns (w_hat [out, in], binary [out, G, g, q] of -1/+1, alpha [out, G, q]); alpha is
    non-negative and, after any refinement, sorted in descending order.
    """
    out_ch, in_ch, g = _groups(w, group_size)
    x = w.detach().to(torch.float32).reshape(-1, g)
    B, A = _greedy(x, qbits)
    if qbits > 1:
        for _ in range(rounds):
            B, A = _refine(x, B, A)
    w_hat = torch.einsum("rgq,rq->rg", B, A).reshape(out_ch, in_ch)
    G = in_ch // g
    return w_hat, B.reshape(out_ch, G, g, qbits), A.reshape(out_ch, G, qbits)


@torch.no_grad()
def dequantize_bcq(binary, alpha, offset=None):
    w = torch.einsum("oigb,oib->oig", binary.to(alpha.dtype), alpha)
    if offset is not None:
        w = w + offset
    return w.reshape(binary.shape[0], -1)


@torch.no_grad()
def to_container(binary, alpha, offset=None):
    """Example layout -> container arrays (numpy): bW uint32 [k/32][q][n] with bit t of word w
    = 1 iff the sign of input channel 32 w + t is +1, alpha float32 [G][q][n], q_bias float32
    [G][n] or None.  k = in_features must be a multiple of 32."""
    out_ch, G, g, q = binary.shape
    k = G * g
    if k % 32 != 0:
        raise ValueError("in_features %d is not a multiple of 32" % k)
    bits = (binary.reshape(out_ch, k, q) > 0).permute(2, 0, 1).contiguous().cpu().numpy()      # [q][n][k]
    packed = np.packbits(bits, axis=-1, bitorder="little")                                      # [q][n][k/8]
    bW = np.ascontiguousarray(packed).view("<u4").transpose(2, 0, 1)                             # [k/32][q][n]
    alpha_c = alpha.permute(1, 2, 0).contiguous().to(torch.float32).cpu().numpy()
    q_bias = None
    if offset is not None:
        q_bias = offset.reshape(out_ch, G).t().contiguous().to(torch.float32).cpu().numpy()
    return dict(bW=np.ascontiguousarray(bW), alpha=alpha_c, q_bias=q_bias, k=k, n=out_ch, q=q, num_groups=G, g=g)


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
