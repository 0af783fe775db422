"""Quantisers and layout converters (host side, torch on the CPU): closed forms and invariants.

The reference's examples hold no fixtures for these steps, and bcq.quantize cannot run without a
CUDA device, so each function is pinned by what the mathematics fixes: the uniform-code identity
of examples/rtn_parameter.py:77-96 checked exhaustively, exact recovery of weights that are
representable, the greedy closed form of examples/bcq.py:105-119, monotone error under
refinement, and agreement of the packed container with the dense weight the oracle rebuilds."""
import os

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


def test_weight_factors_closed_form():
    """examples/bcq.py:52-76 on four weights worked by hand."""
    x = torch.tensor([[1.0, -2.0, 3.0, -4.0]])
    assert Q._weight_factors(x.clone(), 0.0, 1.0, 0.0) is None
    # clipping 0.5: threshold = sorted |w| [int(4*0.5)] = 3; factor = |w|/3 saturated at 1
    wf = Q._weight_factors(x.clone(), 0.0, 0.5, 0.0)
    assert torch.allclose(wf, torch.tensor([[1 / 3, 2 / 3, 1.0, 1.0]]))
    # exponent 2 on |w| / max|w|
    wf = Q._weight_factors(x.clone(), 2.0, 1.0, 0.0)
    assert torch.allclose(wf, torch.tensor([[1 / 16, 4 / 16, 9 / 16, 1.0]]))
    # pruning 0.5: threshold = sorted |w| [2] = 3: |w| <= 3 gets factor 0 and is zeroed
    xx = x.clone()
    wf = Q._weight_factors(xx, 0.0, 1.0, 0.5)
    assert torch.equal(wf, torch.tensor([[0.0, 0.0, 0.0, 1.0]]))
    assert torch.equal(xx, torch.tensor([[0.0, 0.0, 0.0, -4.0]]))


def test_weighted_greedy_and_least_squares():
    gen = torch.Generator().manual_seed(2)
    x = torch.randn(6, 32, generator=gen)
    wf = torch.rand(6, 32, generator=gen) + 0.1
    # one plane: the weighted least-squares scale for b = sign(w) is sum wf |w| / sum wf
    B, A = Q._greedy(x, 1, wf)
    assert torch.allclose(A[:, 0], (wf * x.abs()).sum(1) / wf.sum(1), rtol=1e-6)
    # refinement: for the signs it is given, the new scales satisfy the weighted normal equations
    # B^T diag(wf) (x - B a) = 0 (weights built from sorted positive scales, so |.| and the sort
    # leave them alone), and an unweighted solve does not
    pats = torch.where(torch.rand(6, 32, 3, generator=gen) > 0.5, 1.0, -1.0)
    a_true = torch.tensor([0.9, 0.5, 0.2]).expand(6, 3)
    xw = torch.einsum("rgq,rq->rg", pats, a_true) + 0.05 * torch.randn(6, 32, generator=gen)
    _, A1 = Q._refine(xw, pats, a_true.clone(), wf, use_bst=True)
    resid = xw - torch.einsum("rgq,rq->rg", pats, A1)
    grad = torch.einsum("rgq,rg->rq", pats, wf * resid)
    assert grad.abs().max() < 1e-3
    _, A0 = Q._refine(xw, pats, a_true.clone(), None, use_bst=True)
    resid0 = xw - torch.einsum("rgq,rq->rg", pats, A0)
    assert torch.einsum("rgq,rg->rq", pats, wf * resid0).abs().max() > 1e-2
    # a zero factor everywhere in a group gives scale 0, not NaN
    wz = wf.clone()
    wz[0] = 0.0
    _, Az = Q._greedy(x, 2, wz)
    assert torch.equal(Az[0], torch.zeros(2)) and torch.isfinite(Az).all()


def test_quantize_options():
    gen = torch.Generator().manual_seed(3)
    w = torch.randn(48, 128, generator=gen)
    base, Bb, Ab, kept = Q.quantize(w, 3, rounds=4, group_size=64)
    assert kept.all() and Bb.shape == (48, 2, 64, 3) and Ab.shape == (48, 2, 3)
    w3, B3, A3 = Q.bcq_quantize(w, 3, rounds=4, group_size=64)
    assert torch.equal(w3, base) and torch.equal(B3, Bb) and torch.equal(A3, Ab)
    # transpose: groups along the first dimension = the plain call on w.T
    wt, Bt, At, _ = Q.quantize(w, 3, rounds=4, group_size=16, transpose=True)
    w2, B2, A2, _ = Q.quantize(w.t().contiguous(), 3, rounds=4, group_size=16)
    assert Bt.shape == (128, 3, 16, 3) and torch.equal(Bt, B2) and torch.equal(At, A2) and torch.equal(wt, w2.t())
    # greedy sign assignment: plane 0 is the sign of the weight, plane i the sign of the residual
    wg, Bg, Ag, _ = Q.quantize(w, 3, rounds=3, group_size=64, use_bst=False)
    x = w.reshape(-1, 64)
    Bg2, Ag2 = Bg.reshape(-1, 64, 3), Ag.reshape(-1, 3)
    r = x.clone()
    for i in range(3):
        assert torch.equal(Bg2[:, :, i], torch.where(r >= 0, 1.0, -1.0))
        r -= Bg2[:, :, i] * Ag2[:, i:i + 1]
    # the nearest-level assignment is never worse than the greedy one for the same scales
    assert (base - w).pow(2).sum() <= (wg - w).pow(2).sum() * 1.001
    # pruning: that fraction of the smallest weights is dropped: code 0 in every plane, value 0
    wp, Bp, Ap, keptp = Q.quantize(w, 3, rounds=3, group_size=64, pruning=0.25)
    frac = 1.0 - keptp.float().mean().item()
    assert abs(frac - 0.25) < 0.01
    dropped = ~keptp.reshape(48, 2, 64)
    assert (Bp[dropped] == 0).all() and (Bp[~dropped].abs() == 1).all()
    assert (wp.reshape(48, 2, 64)[dropped] == 0).all()
    assert w.abs().reshape(48, 2, 64)[dropped].max() <= w.abs().reshape(48, 2, 64)[~dropped].min()
    with pytest.raises(ValueError, match="zeros"):
        Q.to_container(Bp, Ap)
    # importance weighting moves error away from the large weights
    we, _, _, _ = Q.quantize(w, 2, rounds=6, group_size=64, exponent=2.0)
    wu, _, _, _ = Q.quantize(w, 2, rounds=6, group_size=64)
    big = w.abs() > w.abs().quantile(0.9)
    assert (we - w)[big].pow(2).mean() < (wu - w)[big].pow(2).mean()


def test_pruned_weights_have_code_zero_on_every_route_and_ties_go_up():
    """Pruned weights (factor 0, value 0) get 0 in every plane whatever the route (greedy only,
    greedy sign assignment, nearest level), as r.sign() of a zero residual gives in
    examples/bcq.py:106; a weight exactly between two levels takes the upper one, as the
    `w < mid` test of examples/bcq.py:177-181 decides."""
    from lutgemm import quantize as qz
    torch.manual_seed(7)
    w = torch.randn(16, 64)
    for rounds, use_bst in ((0, True), (3, False), (3, True)):
        w_hat, binary, alpha, kept = qz.quantize(w, 3, rounds=rounds, group_size=32, pruning=0.3, use_bst=use_bst)
        kept = kept.reshape(binary.shape[:3])
        assert (~kept).any() and kept.any()
        assert bool((binary[~kept] == 0).all()) and bool((binary[kept].abs() == 1).all())
        assert bool((w_hat.reshape(kept.shape)[~kept] == 0).all())
    # levels of alpha = (2, 1) are -3, -1, 1, 3 with midpoints -2, 0, 2.  Four weights sit on the
    # levels and fix the scales; two more sit exactly on midpoints (0 and 2) with a negligible
    # weight in the least squares: they must take the upper levels 1 and 3.
    x = torch.tensor([[3.0, 1.0, -1.0, -3.0, 0.0, 2.0]])
    B = torch.tensor([[[1.0, 1.0], [1.0, -1.0], [-1.0, 1.0], [-1.0, -1.0], [-1.0, 1.0], [1.0, -1.0]]])
    wf = torch.tensor([[1.0, 1.0, 1.0, 1.0, 1e-12, 1e-12]])
    B_new, A_new = qz._refine(x, B, torch.tensor([[2.0, 1.0]]), wf)
    assert torch.allclose(A_new, torch.tensor([[2.0, 1.0]]), atol=1e-4)
    got = (B_new * A_new[:, None, :]).sum(-1)
    assert torch.allclose(got, torch.tensor([[3.0, 1.0, -1.0, -3.0, 1.0, 3.0]]), atol=1e-3)


def test_packer_known_answer_and_round_trip():
    """examples/utils.py:164-183: entry i*N/8 + j of the flattened tensor is bit i of byte j."""
    b = -torch.ones(2, 8)            # N = 16, two bytes
    b[0, 0] = 1                      # flat 0  = 0*2 + 0 -> byte 0 bit 0
    b[0, 3] = 1                      # flat 3  = 1*2 + 1 -> byte 1 bit 1
    b[1, 6] = 1                      # flat 14 = 7*2 + 0 -> byte 0 bit 7
    pb, shape = Q.PACKER.pack(b)
    assert pb.dtype == torch.uint8 and pb.tolist() == [0x81, 0x02] and tuple(shape) == (2, 8)
    assert torch.equal(Q.PACKER.unpack(pb, shape, torch.float32), b)
    gen = torch.Generator().manual_seed(4)
    r = torch.where(torch.rand(3, 4, 16, 2, generator=gen) > 0.5, 1.0, -1.0)
    pr, sh = Q.PACKER.pack(r)
    assert pr.numel() == r.numel() // 8 and torch.equal(Q.PACKER.unpack(pr, sh, torch.float32), r)


@pytest.mark.parametrize("in_ch_wise", [False, True])
def test_parameter_classes_follow_the_example_flow(in_ch_wise):
    """The flow of the reference's examples (examples/rtn_parameter.py:98-112,
    examples/bcq_parameter.py:70-81): RTN compress -> decompress, conversion to BCQ with and
    without packing, BCQ decompress of the converted codes equals the RTN decompress."""
    gen = torch.Generator().manual_seed(6)
    w_org = torch.randn(64, 256, generator=gen)
    w_rtn = Q.RTNParameter(w_org)
    scale, zero, codes, shape = w_rtn.compress(in_ch_wise=in_ch_wise, qbits=4, group_size=32, perchannel=True, sym=False)
    d0 = 256 if in_ch_wise else 64
    assert tuple(shape) == (d0, (64 * 256 // d0) // 32, 32) and scale.shape == (d0, shape[1], 1)
    w_rtn.decompress(scale, zero, codes, shape, in_ch_wise=in_ch_wise)
    assert w_rtn.data.shape == (64, 256)
    assert (w_rtn.data - w_org).abs().max() <= scale.max() * 0.5001
    for packing in (False, True):
        alpha, binary, bshape, offset = w_rtn.convert_bcq_format(scale, zero, codes, qbits=4, do_packing=packing,
                                                                 in_ch_wise=in_ch_wise)
        assert tuple(bshape) == tuple(shape) + (4,)
        assert binary.dtype == (torch.uint8 if packing else torch.float32)
        w_bcq = Q.BCQParameter(w_org)
        w_bcq.decompress(alpha, binary, bshape, offset=offset, do_packing=packing, in_ch_wise=in_ch_wise)
        assert torch.allclose(w_bcq.data, w_rtn.data, atol=1e-5)
    w_bcq = Q.BCQParameter(w_org)
    alpha, binary, bshape = w_bcq.compress(do_packing=True, in_ch_wise=in_ch_wise, qbits=3, rounds=4, group_size=32)
    assert alpha.shape == (d0, shape[1], 3) and binary.numel() == 64 * 256 * 3 // 8
    w_bcq.decompress(alpha, binary, bshape, do_packing=True, in_ch_wise=in_ch_wise)
    assert w_bcq.data.shape == (64, 256) and (w_bcq.data - w_org).abs().mean() < 0.2


def test_rtn_whole_tensor_range():
    """perchannel=False: one (scale, zero) for the whole tensor (examples/utils.py:69-70)."""
    gen = torch.Generator().manual_seed(7)
    w = torch.randn(8, 64, generator=gen)
    scale, zero, codes = Q.rtn_quantize(w, 4, group_size=32, perchannel=False)
    assert scale.shape == (8, 2, 1) and (scale == scale.flatten()[0]).all() and (zero == zero.flatten()[0]).all()
    assert torch.isclose(scale.flatten()[0], (w.max() - w.min()) / 15)
    assert (Q.rtn_dequantize(scale, zero, codes) - w).abs().max() <= scale.flatten()[0] * 0.5001


class _Block(torch.nn.Module):
    def __init__(self, d, f, bias):
        super().__init__()
        self.q_proj = torch.nn.Linear(d, d, bias=bias)
        self.fc1 = torch.nn.Linear(d, f, bias=bias)
        self.fc2 = torch.nn.Linear(f, d, bias=bias)
        self.gate = torch.nn.Linear(d, d)      # not one of the converted names
        self.norm = torch.nn.LayerNorm(d)

    def forward(self, x):
        h = self.norm(x)
        h = x + self.q_proj(h)
        return h + self.fc2(torch.relu(self.fc1(h)))


def test_quantize_model_finds_the_projection_layers():
    torch.manual_seed(8)
    model = torch.nn.Sequential(_Block(64, 128, True), _Block(64, 128, False))
    found = Q.quantize_model(model, qbits=3, group_size=32, method="rtn", to_device=False)
    assert sorted(found) == ["0.fc1", "0.fc2", "0.q_proj", "1.fc1", "1.fc2", "1.q_proj"]
    c = found["1.fc1"]
    assert (c["k"], c["n"], c["q"], c["num_groups"]) == (64, 128, 3, 2) and c["bW"].shape == (2, 3, 128)
    assert isinstance(model[0].fc1, torch.nn.Linear)   # untouched
    with pytest.raises(ValueError, match="no torch.nn.Linear"):
        Q.quantize_model(torch.nn.Sequential(torch.nn.ReLU()), to_device=False)


def test_quant_model_cli_writes_loadable_files(tmp_path, lutgemm, oracle):
    """python -m lutgemm.quant_model, the counterpart of examples/quant_model_rtn.py: a randomly
    initialised OPT saved locally goes in, one packed file per projection layer comes out, and
    a file holds the quantised layer (checked against the oracle's dense weight)."""
    transformers = pytest.importorskip("transformers")
    from lutgemm import quant_model
    cfg = transformers.OPTConfig(vocab_size=64, hidden_size=64, num_hidden_layers=1, ffn_dim=128,
                                 num_attention_heads=2, max_position_embeddings=16, word_embed_proj_dim=64)
    torch.manual_seed(11)
    model = transformers.OPTForCausalLM(cfg)
    src, out = tmp_path / "opt-tiny", tmp_path / "packed"
    model.save_pretrained(src)
    assert quant_model.main(["--model_name_or_path", str(src), "--qbits", "3", "--group_size", "32",
                             "--method", "rtn", "--out_dir", str(out)]) == 0
    files = sorted(f for f in os.listdir(out) if f.endswith(".lutw"))
    assert len(files) == 6 and "model.decoder.layers.0.fc1.lutw" in files
    assert os.path.exists(out / "model.decoder.layers.0.fc1.bias.npy")
    f = lutgemm.unpack_file(str(out / "model.decoder.layers.0.fc1.lutw"))
    assert (f["k"], f["n"], f["q"], f["num_groups"]) == (64, 128, 3, 2) and f["q_bias"] is not None
    w = model.model.decoder.layers[0].fc1.weight.detach().float()
    _, w_hat = Q.quantize_linear(w, 3, 32, "rtn")
    dense = oracle.dense_weight_f64(f["bW"], f["alpha"], f["q_bias"])          # [k][n]
    assert np.abs(dense.T - w_hat.numpy()).max() <= 2e-3 * np.abs(w_hat.numpy()).max() + 1e-4
    with pytest.raises(SystemExit):
        quant_model.main(["--model_name_or_path", str(tmp_path / "missing"), "--out_dir", str(out)])


@pytest.mark.gpu
def test_packed_files_load_into_a_model(tmp_path, lutgemm, device):
    """Offline packing, then loading: the model read from the files computes exactly what the
    model built from the same containers in memory computes."""
    print("case load_packed_model", flush=True)
    torch.manual_seed(12)
    base = torch.nn.Sequential(_Block(256, 512, True), _Block(256, 512, False)).half().float()  # fp16-exact weights
    found = Q.quantize_model(base, qbits=3, group_size=128, method="rtn", to_device=False)
    for name, c in found.items():
        lutgemm.pack_file(str(tmp_path / (name + ".lutw")), c["bW"], c["alpha"], c["k"], c["n"], c["q"],
                          c["num_groups"], c["q_bias"])
    import copy
    a = copy.deepcopy(base).half().to(device)
    b = copy.deepcopy(base).half().to(device)
    from lutgemm.torch_ops import LutLinear
    for name, c in found.items():     # the same containers, straight from memory
        blk, attr = name.split(".")
        lin = getattr(a[int(blk)], attr)
        setattr(a[int(blk)], attr, LutLinear(c, bias=None if lin.bias is None else lin.bias.detach()))
    names = Q.load_packed_model(b, str(tmp_path))
    assert sorted(names) == sorted(found)
    x = torch.randn(3, 256, device=device, dtype=torch.float16)
    with torch.no_grad():
        assert torch.equal(a(x), b(x))
    with pytest.raises(ValueError, match="no packed-weight file"):
        Q.load_packed_model(copy.deepcopy(base), str(tmp_path / "nothing-here"))


@pytest.mark.gpu
def test_quantize_model_on_device(lutgemm, device):
    """The converted model computes what the same model with the dequantised weights computes:
    decode-sized inputs take the LUT kernel, larger ones the dense route."""
    print("case quantize_model", flush=True)
    from lutgemm.torch_ops import LutLinear
    torch.manual_seed(9)
    model = torch.nn.Sequential(_Block(256, 512, True), _Block(256, 512, False)).half().to(device)
    ref = torch.nn.Sequential(_Block(256, 512, True), _Block(256, 512, False)).half().to(device)
    ref.load_state_dict(model.state_dict())
    for blk in ref:
        for name in ("q_proj", "fc1", "fc2"):
            lin = getattr(blk, name)
            _, w_hat = Q.quantize_linear(lin.weight.detach().float(), 4, 64, "rtn")
            lin.weight.data.copy_(w_hat.half())
    Q.quantize_model(model, qbits=4, group_size=64, method="rtn")
    assert all(isinstance(getattr(b, nm), LutLinear) for b in model for nm in ("q_proj", "fc1", "fc2"))
    assert isinstance(model[0].gate, torch.nn.Linear)
    for rows in (1, 2, 5, 32):
        x = torch.randn(rows, 256, device=device, dtype=torch.float16)
        with torch.no_grad():
            y, want = model(x), ref(x)
        err = (y.float() - want.float()).abs().max().item()
        assert err <= 0.02 * want.float().abs().max().item() + 0.02, (rows, err)


@pytest.mark.gpu
def test_opt_decoder_quantised_end_to_end(lutgemm, device):
    """A randomly initialised OPT decoder (the model family the reference's walkers convert,
    examples/quant_model_rtn.py:34): every q/k/v/out projection and both MLP layers replaced by
    packed weights; prefill and one cached decode step give the logits of the same model run
    with the dequantised weights."""
    transformers = pytest.importorskip("transformers")
    from lutgemm.torch_ops import LutLinear
    print("case OPT decoder", flush=True)
    cfg = transformers.OPTConfig(vocab_size=512, hidden_size=256, num_hidden_layers=2, ffn_dim=1024,
                                 num_attention_heads=4, max_position_embeddings=64, word_embed_proj_dim=256)
    torch.manual_seed(10)
    model = transformers.OPTForCausalLM(cfg).eval().half().to(device)
    ref = transformers.OPTForCausalLM(cfg).eval().half().to(device)
    ref.load_state_dict(model.state_dict())
    for name, mod in ref.named_modules():
        if isinstance(mod, torch.nn.Linear) and any(x in name.split(".")[-1] for x in Q.DEFAULT_LAYERS):
            _, w_hat = Q.quantize_linear(mod.weight.detach().float(), 4, 128, "rtn")
            mod.weight.data.copy_(w_hat.half())
    Q.quantize_model(model, qbits=4, group_size=128, method="rtn")
    converted = [n for n, m in model.named_modules() if isinstance(m, LutLinear)]
    assert len(converted) == 12 and isinstance(model.lm_head, torch.nn.Linear)
    ids = torch.randint(0, 512, (1, 6), device=device)
    nxt = torch.randint(0, 512, (1, 1), device=device)
    with torch.no_grad():
        a = model(ids, use_cache=True)
        b = ref(ids, use_cache=True)
        a1 = model(nxt, past_key_values=a.past_key_values, use_cache=True)   # one row: the LUT kernel
        b1 = ref(nxt, past_key_values=b.past_key_values, use_cache=True)
        long_ids = torch.randint(0, 512, (2, 12), device=device)             # 24 rows: dense route
        c, d = model(long_ids).logits, ref(long_ids).logits
    for got, want, what in ((a.logits, b.logits, "prefill"), (a1.logits, b1.logits, "decode"), (c, d, "batch")):
        err = (got.float() - want.float()).abs().max().item()
        assert err <= 0.02 * want.float().abs().max().item() + 0.02, (what, err)
    assert torch.equal(a1.logits.argmax(-1), b1.logits.argmax(-1))


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
