"""rz_sgd_step / rz_adam_step (rzlinear_amd.optim.FusedSGD / FusedAdam) against torch.optim on the
same values: the update rules are torch's, so several steps must agree to fp32 rounding; 16-bit
parameters with an fp32 master copy must be the rounded fp32 trajectory; a gradient in an fp32
main_grad buffer (what fuse_grad_accumulation fills) is picked up."""
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def _grads(n, steps, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn((n,), generator=g).cuda() * (0.5 + i) for i in range(steps)]


SGD_CASES = [dict(lr=0.1), dict(lr=0.05, momentum=0.9), dict(lr=0.05, momentum=0.9, dampening=0.1, weight_decay=0.01),
             dict(lr=0.02, momentum=0.8, nesterov=True, weight_decay=0.1)]
ADAM_CASES = [dict(lr=1e-2), dict(lr=3e-3, betas=(0.8, 0.95), eps=1e-6, weight_decay=0.05),
              dict(lr=3e-3, weight_decay=0.1, decoupled_weight_decay=True)]
_id = lambda d: ",".join("%s=%s" % kv for kv in d.items())


@pytest.mark.parametrize("kw", SGD_CASES, ids=_id)
def test_fused_sgd_follows_torch_sgd(kw):
    from rzlinear_amd.optim import FusedSGD
    n, steps = 70001, 5
    _say("fused sgd", kw)
    w0 = torch.randn((n,), generator=torch.Generator().manual_seed(3)).cuda()
    a, b = torch.nn.Parameter(w0.clone()), torch.nn.Parameter(w0.clone())
    ours, ref = FusedSGD([a], **kw), torch.optim.SGD([b], **kw)
    for g in _grads(n, steps, 5):
        a.grad, b.grad = g.clone(), g.clone()
        ours.step()
        ref.step()
        torch.cuda.synchronize()
        assert torch.allclose(a.detach(), b.detach(), rtol=2e-6, atol=2e-6 * float(b.detach().abs().max()))


@pytest.mark.parametrize("kw", ADAM_CASES, ids=_id)
def test_fused_adam_follows_torch_adam(kw):
    from rzlinear_amd.optim import FusedAdam
    n, steps = 70001, 6
    _say("fused adam", kw)
    w0 = torch.randn((n,), generator=torch.Generator().manual_seed(4)).cuda()
    a, b = torch.nn.Parameter(w0.clone()), torch.nn.Parameter(w0.clone())
    ours = FusedAdam([a], **kw)
    tkw = dict(kw)
    decoupled = tkw.pop("decoupled_weight_decay", False)
    ref = (torch.optim.AdamW if decoupled else torch.optim.Adam)([b], **tkw)
    for g in _grads(n, steps, 6):
        a.grad, b.grad = g.clone(), g.clone()
        ours.step()
        ref.step()
        torch.cuda.synchronize()
        assert torch.allclose(a.detach(), b.detach(), rtol=1e-5, atol=1e-5 * float(b.detach().abs().max()))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=lambda d: str(d).split(".")[-1])
def test_master_weights_carry_small_updates_of_16_bit_parameters(dtype):
    """With an fp32 master copy the 16-bit parameter is the rounded fp32 trajectory; the gradient
    comes from an fp32 main_grad buffer and is scaled by grad_scale."""
    from rzlinear_amd.optim import FusedAdam, FusedSGD
    n, steps = 40000, 8
    _say("master weights", dtype)
    w0 = torch.randn((n,), generator=torch.Generator().manual_seed(7)).to(dtype)
    for make, tmake in ((lambda ps: FusedSGD(ps, lr=1e-3, momentum=0.9, master_weights=True, grad_scale=0.5),
                         lambda ps: torch.optim.SGD(ps, lr=1e-3, momentum=0.9)),
                        (lambda ps: FusedAdam(ps, lr=1e-4, master_weights=True, grad_scale=0.5),
                         lambda ps: torch.optim.Adam(ps, lr=1e-4))):
        a = torch.nn.Parameter(w0.clone().cuda())
        a.main_grad = torch.zeros((n,), dtype=torch.float32, device="cuda")
        b = torch.nn.Parameter(w0.float().cuda())
        ours, ref = make([a]), tmake([b])
        for g in _grads(n, steps, 8):
            a.main_grad.copy_(g)
            b.grad = g * 0.5
            ours.step()
            ref.step()
        torch.cuda.synchronize()
        assert torch.equal(a.detach(), ours.state[a]["master"].to(dtype))
        assert torch.allclose(ours.state[a]["master"], b.detach(), rtol=1e-5, atol=1e-6)
        # without the master copy most of these updates are below the 16-bit spacing
        assert float((a.detach().float() - w0.float().cuda()).abs().max()) > 0
        ours.zero_grad()
        assert float(a.main_grad.abs().max()) == 0.0


def test_layers_sharing_a_parameter_train_with_the_fused_step(oracle):
    """Two layers on one hashed_weight with fuse_grad_accumulation, FusedSGD reading main_grad:
    one step equals hashed_weight - lr * (sum of the layers' oracle gradients)."""
    import numpy as np
    from helpers import SEED_CONSTANTS
    from rzlinear_amd import RzLinear
    from rzlinear_amd.optim import FusedSGD
    torch.manual_seed(0)
    K, N, M = 256, 192, 96
    first = RzLinear(K, N, compress_ratio=0.2, bias=False, dtype=torch.float32, block_size_k=64, block_size_n=64,
                     fuse_grad_accumulation=True).cuda()
    second = RzLinear(K, N, hashed_weight=first._hashed_weight, seed=7, bias=False, dtype=torch.float32,
                      block_size_k=64, block_size_n=64, fuse_grad_accumulation=True).cuda()
    hw = first._hashed_weight
    assert second._hashed_weight is hw
    hw.main_grad = torch.zeros_like(hw, dtype=torch.float32)
    x1, x2 = torch.randn(M, K, device="cuda"), torch.randn(M, K, device="cuda")
    dy1, dy2 = torch.randn(M, N, device="cuda"), torch.randn(M, N, device="cuda")
    before = hw.detach().double().cpu().numpy()
    opt = FusedSGD([hw], lr=0.25)
    first(x1).backward(dy1)
    second(x2).backward(dy2)
    opt.step()
    torch.cuda.synchronize()
    H = hw.numel()
    f64 = lambda t: t.double().cpu().numpy()
    R1 = [int(v) for v in first._random_numbers.tolist()]
    R2 = [int(v) for v in second._random_numbers.tolist()]
    g = oracle.weight_grad(f64(x1), f64(dy1), H, 64, 64, R1, first._init_factor) + \
        oracle.weight_grad(f64(x2), f64(dy2), H, 64, 64, R2, second._init_factor)
    want = before - 0.25 * g
    assert np.abs(f64(hw.detach()) - want).max() <= 1e-4 * np.abs(want).max()
