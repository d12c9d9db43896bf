"""GPU parity of the training-mode batch norm kernels (through libtsmi.so's C ABI) against
torch's batch norm evaluated in fp64 on the same data.

Tolerances, relative to the RMS of the reference result: 1e-5 for fp32, 2e-3 for fp16, 1.6e-2
for bf16 (one rounding of the output type plus the fp32 sums)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.float16: 2e-3, torch.bfloat16: 1.6e-2}


def rel(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return float((a - b).norm() / (b.norm() + 1e-30))


def reference(x, w, b, rm, rv, momentum, eps, dy):
    """torch's own batch norm in fp64 on the values the kernels see."""
    xd = x.double().requires_grad_(True)
    wd = w.double().requires_grad_(True) if w is not None else None
    bd = b.double().requires_grad_(True) if b is not None else None
    rmd, rvd = (rm.double().clone(), rv.double().clone()) if rm is not None else (None, None)
    y = torch.nn.functional.batch_norm(xd, rmd, rvd, wd, bd, True, momentum, eps)
    y.backward(dy.double())
    return y.detach(), xd.grad, (wd.grad if wd is not None else None), (bd.grad if bd is not None else None), rmd, rvd


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("n,c", [(2, 8), (1000, 32), (4099, 96), (90001, 64), (777, 256), (50, 2048)])
def test_batch_norm_kernels_match_torch_fp64(dtype, n, c):
    from torchsparse_amd import backend
    if dtype == torch.float32 and c == 2048:
        pytest.skip("2048 fp32 channels are 512 pieces: beyond the kernels' 256")
    g = torch.Generator(device="cuda").manual_seed(n + c)
    # a column mean far from zero next to a small spread: what the shifted sums are for
    x = (torch.randn(n, c, device="cuda", generator=g) * 0.5 + torch.linspace(-30, 30, c, device="cuda")).to(dtype)
    w = (torch.rand(c, device="cuda", generator=g) + 0.5).to(dtype)
    b = torch.randn(c, device="cuda", generator=g).to(dtype)
    rm = torch.randn(c, device="cuda", generator=g).to(dtype)
    rv = (torch.rand(c, device="cuda", generator=g) + 0.5).to(dtype)
    dy = torch.randn(n, c, device="cuda", generator=g).to(dtype)
    want_y, want_dx, want_dw, want_db, want_rm, want_rv = reference(x, w, b, rm, rv, 0.1, 1e-5, dy)
    assert backend.bn_supported(x, w, b, rm, rv)
    rm1, rv1 = rm.clone(), rv.clone()
    y, mean, invstd = backend.bn_forward_train(x, w, b, rm1, rv1, 0.1, 1e-5)
    dx, dw, db = backend.bn_backward(dy, x, w, mean, invstd)
    tol = TOL[dtype]
    assert rel(y, want_y) < tol
    # dx = w * invstd * (dy - mean(dy) - xhat * mean(dy * xhat)) cancels almost completely for a
    # handful of rows: the error is measured against the size of the terms, not of their difference
    terms = (w.double() * invstd.double() * dy.double()).cpu().norm()
    assert float((dx.double().cpu() - want_dx.cpu()).norm() / terms) < tol * 1.5
    assert rel(dw, want_dw) < max(tol, 1e-4) and rel(db, want_db) < max(tol, 1e-4)  # fp32 sums, stored as w's type
    assert rel(rm1, want_rm) < tol and rel(rv1, want_rv) < tol
    assert rel(mean, x.double().mean(0)) < 1e-6
    assert rel(invstd, 1 / torch.sqrt(x.double().var(0, unbiased=False) + 1e-5)) < 1e-4
    # the same bits on every run
    y2, mean2, invstd2 = backend.bn_forward_train(x, w, b, rm.clone(), rv.clone(), 0.1, 1e-5)
    dx2, dw2, db2 = backend.bn_backward(dy, x, w, mean2, invstd2)
    for a, b_ in ((y, y2), (mean, mean2), (invstd, invstd2), (dx, dx2), (dw, dw2), (db, db2)):
        assert torch.equal(a, b_)


def test_batch_norm_module_uses_the_kernels_in_training_and_torch_otherwise(monkeypatch):
    import torchsparse_amd as ts
    from torchsparse_amd import backend
    from torchsparse_amd import nn as spnn
    torch.manual_seed(0)
    n, c = 3000, 64
    coords = torch.cat([torch.zeros(n, 1, dtype=torch.int32), torch.arange(n, dtype=torch.int32).view(-1, 1).repeat(1, 3)], 1).cuda()
    feats = (torch.randn(n, c, device="cuda") * 2 + 3).half()
    calls = []
    real = backend.bn_forward_train
    monkeypatch.setattr(backend, "bn_forward_train", lambda *a: (calls.append(1), real(*a))[1])
    ours, theirs = spnn.BatchNorm(c).cuda().half(), torch.nn.BatchNorm1d(c).cuda().half()
    with torch.no_grad():
        ours.weight.uniform_(0.5, 1.5), ours.bias.normal_()
        theirs.weight.copy_(ours.weight), theirs.bias.copy_(ours.bias)
    xa, xb = feats.clone().requires_grad_(True), feats.clone().requires_grad_(True)
    ya = ours(ts.SparseTensor(xa, coords)).feats
    yb = theirs(xb)
    assert calls == [1]
    (ya.float() ** 2).mean().backward()
    (yb.float() ** 2).mean().backward()
    assert rel(ya, yb) < 3e-3 and rel(xa.grad, xb.grad) < 5e-3
    assert rel(ours.weight.grad, theirs.weight.grad) < 5e-3 and rel(ours.bias.grad, theirs.bias.grad) < 5e-3
    assert rel(ours.running_mean, theirs.running_mean) < 2e-3 and rel(ours.running_var, theirs.running_var) < 2e-3
    assert int(ours.num_batches_tracked) == 1
    ours.eval(), theirs.eval()
    assert rel(ours(ts.SparseTensor(feats, coords)).feats, theirs(feats)) < 3e-3
    assert calls == [1]  # evaluation mode is torch's
    # 4 channels (a network's input) are not a 16-byte piece: torch again
    small = spnn.BatchNorm(4).cuda().half().train()
    small(ts.SparseTensor(feats[:, :4].contiguous(), coords))
    assert calls == [1]
