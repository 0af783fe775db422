"""The PyTorch operator and LutLinear on the GPU: parity with the oracle, the dense route for
large batches, and replay from a captured HIP graph."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _layer(seed, out_f=320, in_f=1024, bias=True):
    gen = torch.Generator().manual_seed(seed)
    lin = torch.nn.Linear(in_f, out_f, bias=bias)
    with torch.no_grad():
        lin.weight.copy_(torch.randn(out_f, in_f, generator=gen) * 0.03)
        if bias:
            lin.bias.copy_(torch.randn(out_f, generator=gen) * 0.1)
    return lin, gen


@pytest.mark.parametrize("method,qbits", [("rtn", 4), ("bcq", 3)])
def test_lut_linear_matches_oracle(lutgemm, oracle, device, method, qbits):
    from gpu_util import assert_within_tolerance
    from lutgemm import quantize, torch_ops
    print("case LutLinear", method, qbits, flush=True)
    lin, gen = _layer(1)
    c, w_hat = quantize.quantize_linear(lin.weight.detach(), qbits, 128, method, rounds=5)
    layer = torch_ops.LutLinear(c, bias=lin.bias.detach())
    x = torch.randn(2, 3, 1024, generator=gen).to(torch.float16)
    y = layer(x.to(device))
    assert y.shape == (2, 3, 320) and y.dtype == torch.float16
    a16 = c["alpha"].astype(np.float16)
    z16 = c["q_bias"].astype(np.float16) if c["q_bias"] is not None else None
    truth = oracle.matvec_f64(c["bW"], a16, z16, x.reshape(-1, 1024).numpy())
    got = torch.ops.lutgemm.matvec(x.to(device), layer.handle).cpu().numpy().reshape(-1, 320)
    assert_within_tolerance(got, truth, "operator")
    want = truth + lin.bias.detach().to(torch.float16).double().numpy()
    assert np.abs(y.cpu().double().numpy().reshape(-1, 320) - want).max() <= 2e-2


def test_large_batches_take_the_dense_route(lutgemm, oracle, device):
    from lutgemm import quantize, torch_ops
    lin, gen = _layer(2, bias=False)
    c, _ = quantize.quantize_linear(lin.weight.detach(), 4, 128, "rtn")
    layer = torch_ops.LutLinear(c, dense_threshold=8)
    x = torch.randn(40, 1024, generator=gen).to(torch.float16)
    y_dense = layer(x.to(device))                       # 40 rows > threshold: dequantise + GEMM
    # by default the layer keeps no dense copy: the weight is rebuilt per call in the scratch buffer
    # all layers of the stream share, which only grows (what the reference's scratch singleton does)
    assert layer._dense is None
    scratch = torch_ops.dense_scratch(320 * 1024, layer.device, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    shared = scratch.view(320, 1024).clone()            # W^T [n][k]
    small = torch_ops.LutLinear(quantize.quantize_linear(lin.weight.detach()[:64], 4, 128, "rtn")[0], dense_threshold=8)
    y_small = small(x.to(device))
    assert torch_ops.dense_scratch(1, layer.device, torch.cuda.current_stream().cuda_stream).data_ptr() == scratch.data_ptr()
    assert torch.allclose(y_small.float(), y_dense[:, :64].float(), atol=2e-2, rtol=0)   # another GEMM shape
    assert torch.equal(layer(x.to(device)), y_dense)     # rebuilt after another layer used the scratch
    kept = torch_ops.LutLinear(c, dense_threshold=8, keep_dense=True)
    assert torch.equal(kept(x.to(device)), y_dense)
    assert kept._dense is not None and kept._dense.shape == (320, 1024) and torch.equal(kept._dense, shared)
    layer._dense = shared                               # for the checks below
    y_lut = torch.ops.lutgemm.matvec(x.to(device), layer.handle)
    # the dense weight is the oracle's dense weight rounded to fp16
    a16 = c["alpha"].astype(np.float16)
    z16 = c["q_bias"].astype(np.float16)
    dense = oracle.dense_weight_f64(c["bW"], a16, z16)
    assert np.array_equal(layer._dense.cpu().numpy(), dense.T.astype(np.float16))
    truth = x.double().numpy() @ dense
    assert np.abs(y_lut.cpu().double().numpy() - truth).max() <= 1e-2
    assert np.abs(y_dense.cpu().double().numpy() - truth).max() <= 3e-2   # fp16 weight + library GEMM


@pytest.mark.parametrize("rows", [2, 5])   # the two-row table kernel and the batch kernel
def test_operator_replays_from_a_hip_graph(lutgemm, device, rows):
    from lutgemm import quantize, torch_ops
    lin, gen = _layer(3, bias=False)
    c, _ = quantize.quantize_linear(lin.weight.detach(), 3, 128, "bcq", rounds=2)
    layer = torch_ops.LutLinear(c)
    xs = [torch.randn(rows, 1024, generator=gen).to(torch.float16).to(device) for _ in range(3)]
    eager = [layer(x).clone() for x in xs]
    static_x = xs[0].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        layer(static_x)
        side.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            static_y = layer(static_x)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for rep in range(2):
        for x, want in zip(xs, eager):
            static_x.copy_(x)
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_y, want), "replay %d differs from the eager result" % rep


def test_operator_argument_checks(lutgemm, device):
    from lutgemm import quantize, torch_ops
    lin, _ = _layer(4, bias=False)
    c, _ = quantize.quantize_linear(lin.weight.detach(), 2, 128, "rtn")
    layer = torch_ops.LutLinear(c)
    with pytest.raises(Exception):
        torch.ops.lutgemm.matvec(torch.zeros(1, 1024, dtype=torch.float32, device=device), layer.handle)
    with pytest.raises(Exception):
        torch.ops.lutgemm.matvec(torch.zeros(1, 512, dtype=torch.float16, device=device), layer.handle)
    with pytest.raises(Exception):
        torch.ops.lutgemm.matvec(torch.zeros(1, 1024, dtype=torch.float16, device=device), 10 ** 9)


def test_default_dense_threshold_follows_the_weight(lutgemm, device):
    """The packed route is kept for as many passes of 16 rows as cost less than the dense route:
    more of them when the dense weight has to be rebuilt per call than when the layer keeps it."""
    from lutgemm import quantize, torch_ops
    print("case default dense threshold", flush=True)
    lin, _ = _layer(5, out_f=64, in_f=512, bias=False)
    for qbits, g, want, want_kept in ((2, 128, 80, 32), (4, 128, 48, 16), (3, 64, 64, 16), (1, 32, 80, 32), (5, 128, 48, 16),
                                      (8, 128, 48, 2)):
        c, _ = quantize.quantize_linear(lin.weight.detach(), qbits, g, "rtn", rounds=0)
        layer = torch_ops.LutLinear(c)
        assert layer.dense_threshold == want, (qbits, g, layer.dense_threshold)
        kept = torch_ops.LutLinear(c, keep_dense=True)
        assert kept.dense_threshold == want_kept, (qbits, g, kept.dense_threshold)
        kept.weight.close()
        assert torch_ops.LutLinear(c, dense_threshold=7).dense_threshold == 7
        layer.weight.close()
