"""Quantisers and layout converters (host side, torch on the CPU): closed forms and invariants.

The reference's examples hold no fixtures for these steps, and bcq.quantize cannot run without a
CUDA device, so each function is pinned by what the mathematics fixes: the uniform-code identity
of examples/rtn_parameter.py:77-96 checked exhaustively, exact recovery of weights that are
representable, the greedy closed form of examples/bcq.py:105-119, monotone error under
refinement, and agreement of the packed container with the dense weight the oracle rebuilds."""
import numpy as np
import pytest
import torch

from lutgemm import quantize as Q


def test_rtn_reproduces_exact_levels():
    # a group that already holds the 16 levels of a 4-bit grid (zero included) comes back exactly
    scale_true, zero_true = 0.125, 5
    levels = scale_true * (torch.arange(16, dtype=torch.float32) - zero_true)
    w = levels[torch.randperm(16, generator=torch.Generator().manual_seed(0))].repeat(3, 8)  # [3, 128]
    scale, zero, codes = Q.rtn_quantize(w, 4, group_size=128)
    assert scale.shape == (3, 1, 1) and codes.shape == (3, 1, 128)
    assert torch.allclose(scale, torch.full_like(scale, scale_true)) and torch.all(zero == zero_true)
    assert torch.equal(Q.rtn_dequantize(scale, zero, codes), w)
    assert codes.min() == 0 and codes.max() == 15


@pytest.mark.parametrize("qbits,g,sym", [(4, 128, False), (3, 64, False), (2, 32, True), (4, 256, True), (8, 128, False)])
def test_rtn_error_bound_and_range(qbits, g, sym):
    gen = torch.Generator().manual_seed(qbits * 100 + g)
    w = torch.randn(24, 512, generator=gen) * 0.05
    scale, zero, codes = Q.rtn_quantize(w, qbits, g, sym=sym)
    assert codes.min() >= 0 and codes.max() <= 2 ** qbits - 1
    err = (Q.rtn_dequantize(scale, zero, codes) - w).reshape(24, 512 // g, g).abs()
    # round to nearest on a grid that covers the group's range: at most half a step off
    assert torch.all(err <= scale / 2 + 1e-7)
    if sym:
        assert torch.all(zero == 2 ** qbits / 2)


@pytest.mark.parametrize("qbits,sym", [(3, False), (4, False), (4, True)])
def test_rtn_range_search_never_worse_in_its_own_norm(qbits, sym):
    """mse=True tries the full range first (shrink factor 1), so per group its sum |error|^norm
    cannot exceed the plain min/max result; with outliers stretching the range it is better overall."""
    gen = torch.Generator().manual_seed(17)
    w = torch.randn(32, 256, generator=gen) * 0.02
    w[:, ::64] *= 8.0                                   # outliers that stretch the min/max range
    plain = Q.rtn_quantize(w, qbits, 128, sym=sym)
    tuned = Q.rtn_quantize(w, qbits, 128, sym=sym, mse=True)
    def err(r):
        return (Q.rtn_dequantize(*r) - w).reshape(32, 2, 128).abs().pow(2.4).sum(-1)
    e0, e1 = err(plain), err(tuned)
    assert torch.all(e1 <= e0 * (1 + 1e-6))
    assert e1.sum() < e0.sum() * 0.97 and (e1 < e0 * 0.95).any()
    assert tuned[2].min() >= 0 and tuned[2].max() <= 2 ** qbits - 1
    assert torch.all(tuned[0] <= plain[0] * (1 + 1e-6))  # the range only shrinks


@pytest.mark.parametrize("qbits", [1, 2, 3, 4, 8])
def test_rtn_to_bcq_identity_over_all_codes(qbits):
    # every code value, several (scale, zero): sum_i alpha_i s_i + offset == scale (c - zero)
    codes = torch.arange(2 ** qbits, dtype=torch.int32).reshape(1, 1, -1).repeat(4, 2, 1)
    scale = torch.tensor([0.5, 0.03125, 1.75, 0.0078125]).reshape(4, 1, 1).repeat(1, 2, 1).double()
    zero = torch.tensor([0.0, 3.0, 7.0, 200.0]).reshape(4, 1, 1).repeat(1, 2, 1).double()
    alpha, binary, offset = Q.rtn_to_bcq(scale, zero, codes, qbits)
    assert alpha.shape == (4, 2, qbits) and binary.shape == (4, 2, 2 ** qbits, qbits) and offset.shape == (4, 2, 1)
    assert set(binary.unique().tolist()) <= {-1.0, 1.0}
    # planes are least significant first with alpha_i = scale 2^i / 2
    assert torch.equal(alpha[..., 0], scale[..., 0] / 2)
    if qbits > 1:
        assert torch.equal(alpha[..., 1], scale[..., 0])
    want = (scale * (codes.double() - zero)).reshape(4, -1)
    assert torch.equal(Q.dequantize_bcq(binary, alpha, offset), want)  # exact: powers of two


def test_bcq_greedy_closed_form():
    gen = torch.Generator().manual_seed(3)
    w = torch.randn(6, 256, generator=gen)
    w[0, 0] = 0.0  # a zero weight gets sign +1
    w_hat, B, A = Q.bcq_quantize(w, 3, rounds=0, group_size=64)
    x = w.reshape(-1, 64)
    r = x.clone()
    for i in range(3):
        b = torch.where(r >= 0, 1.0, -1.0)
        a = r.abs().mean(dim=1, keepdim=True)
        assert torch.equal(B.reshape(-1, 64, 3)[:, :, i], b)
        assert torch.allclose(A.reshape(-1, 3)[:, i], a[:, 0])
        r = r - a * b
    assert torch.allclose(w_hat, w - r.reshape(6, 256), atol=1e-6)
    # one plane: the scale is the mean magnitude, the error is orthogonal to the sign vector
    w1, B1, A1 = Q.bcq_quantize(w, 1, rounds=5, group_size=256)
    assert torch.allclose(A1[:, 0, 0], w.abs().mean(dim=1))
    assert torch.allclose(((w - w1) * B1[:, 0, :, 0]).sum(dim=1), torch.zeros(6), atol=1e-4)


def test_bcq_refinement_monotone_sorted_and_exact_on_representable_weights():
    gen = torch.Generator().manual_seed(11)
    w = torch.randn(16, 512, generator=gen) * 0.02
    prev = None
    for rounds in (0, 1, 2, 4, 8, 15):
        w_hat, B, A = Q.bcq_quantize(w, 3, rounds=rounds, group_size=128)
        err = ((w - w_hat) ** 2).sum().item()
        if prev is not None:
            assert err <= prev * (1 + 1e-5)
        prev = err
        assert torch.all(A >= 0)
        if rounds:
            assert torch.all(A[..., :-1] >= A[..., 1:])
        assert torch.allclose(Q.dequantize_bcq(B, A), w_hat, atol=1e-6)
        assert set(B.unique().tolist()) <= {-1.0, 1.0}
    # better than uniform rounding to the same number of levels would suggest: a sanity bound
    assert prev < ((w - w.mean()) ** 2).sum().item() * 0.1
    # weights that are exactly sum_i alpha_i s_i are recovered exactly
    signs = torch.where(torch.rand(8, 128, 3, generator=gen) < 0.5, -1.0, 1.0)
    alpha = torch.tensor([1.0, 0.5, 0.25])
    wrep = (signs * alpha).sum(-1)
    w_hat, B, A = Q.bcq_quantize(wrep, 3, rounds=10, group_size=128)
    assert torch.allclose(w_hat, wrep, atol=1e-5)
    assert torch.allclose(A.reshape(-1, 3), alpha.expand(8, 3), atol=1e-5)


@pytest.mark.parametrize("method,qbits,g", [("rtn", 4, 128), ("rtn", 3, 64), ("bcq", 3, 128), ("bcq", 2, 32)])
def test_container_matches_dequantised_weight(oracle, lutgemm, method, qbits, g):
    """to_container's bit packing, transposes and offset placement: the dense weight the oracle
    rebuilds from the container (W[k][n], fp16 scales) equals the quantiser's own dequantised
    weight transposed, up to the fp16 rounding of the scales."""
    gen = torch.Generator().manual_seed(qbits * 7 + g)
    w = torch.randn(40, 256, generator=gen) * 0.03          # [out=40, in=256]
    c, w_hat = Q.quantize_linear(w, qbits, group_size=g, method=method, rounds=4)
    assert c["bW"].shape == (256 // 32, qbits, 40) and c["bW"].dtype == np.uint32
    assert c["alpha"].shape == (256 // g, qbits, 40)
    assert (c["q_bias"] is not None) == (method == "rtn")
    a16 = c["alpha"].astype(np.float16)
    z16 = c["q_bias"].astype(np.float16) if c["q_bias"] is not None else None
    dense = oracle.dense_weight_f64(c["bW"], a16, z16)       # [k][n]
    tol = 2.0 ** -10 * (np.abs(c["alpha"]).sum(axis=1).max() + (0 if z16 is None else np.abs(c["q_bias"]).max()))
    assert np.abs(dense - w_hat.numpy().T.astype(np.float64)).max() <= tol
    # and the host packer accepts it
    signs, scales = lutgemm.pack_host(c["bW"], a16.view(np.uint16), None if z16 is None else z16.view(np.uint16),
                                      c["k"], c["n"], c["q"], c["num_groups"])
    bW2, a2, z2 = lutgemm.unpack_host(signs, scales, c["k"], c["n"], c["q"], c["num_groups"], z16 is not None)
    assert np.array_equal(bW2, c["bW"])


def test_bit_order_of_container_words():
    # one +1 sign at input channel 37 of output 2, plane 1: bit 5 of word 1
    binary = -torch.ones(3, 1, 64, 2)
    binary[2, 0, 37, 1] = 1.0
    alpha = torch.ones(3, 1, 2)
    c = Q.to_container(binary, alpha)
    want = np.zeros((2, 2, 3), np.uint32)
    want[1, 1, 2] = 1 << 5
    assert np.array_equal(c["bW"], want)


@pytest.mark.gpu
@pytest.mark.parametrize("method,qbits,g", [("rtn", 4, 128), ("bcq", 3, 128), ("rtn", 3, 64)])
def test_quantised_linear_on_device(lutgemm, oracle, device, method, qbits, g):
    """A quantised linear layer end to end: y = x @ w_hat.T through the packed container."""
    from gpu_util import assert_within_tolerance, run_matvec
    print("case quantised linear", method, qbits, g, flush=True)
    gen = torch.Generator().manual_seed(5)
    w = torch.randn(300, 1024, generator=gen) * 0.03
    c, w_hat = Q.quantize_linear(w, qbits, group_size=g, method=method, rounds=6)
    W = lutgemm.BCQWeight(c["bW"], c["alpha"], c["k"], c["n"], c["q"], c["num_groups"], c["q_bias"])
    x = (torch.randn(3, 1024, generator=gen)).to(torch.float16).numpy()
    y = run_matvec(lutgemm, W, x, device)
    a16 = c["alpha"].astype(np.float16)
    z16 = c["q_bias"].astype(np.float16) if c["q_bias"] is not None else None
    truth = oracle.matvec_f64(c["bW"], a16, z16, x)
    assert_within_tolerance(y, truth, "quantised linear %s q=%d g=%d" % (method, qbits, g))
    # and close to the layer the quantiser describes (scales rounded to fp16 in the container)
    ref = x.astype(np.float64) @ w_hat.numpy().T.astype(np.float64)
    assert np.abs(y.astype(np.float64) - ref).max() <= 0.05 * np.abs(ref).max() + 0.02
    W.close()
