"""The reference's CPU-runnable path, restated with torch — TEST/BENCH INFRASTRUCTURE ONLY.

"Hash-gather W, then torch.matmul": the design of the reference's own test oracles
(python/tests/test_rz_linear.py:21-33 for W, :77-90 for the scatter-add of the dense weight
gradient), with the two-level hash of the kernels (python/rz_linear/impl/RzLinearForward.py:316).
Used as the timed CPU baseline of bench.py and by the smoke check; never by the product."""
import time

import torch

from . import rz_oracle


class CpuPath:
    """fp32 forward + backward of one RzLinear layer on the host cores."""

    def __init__(self, K, N, H, BK, BN, R, init_factor=1.0):
        self.K, self.N, self.H, self.f = K, N, H, float(init_factor)
        # built once, outside any timer
        self.index_map = torch.from_numpy(rz_oracle.index_map(K, N, H, BK, BN, R))
        self.flat_index = self.index_map.reshape(-1)

    def forward(self, x, hw):
        w = hw[self.index_map]
        return torch.matmul(x, w) * self.f

    def backward(self, x, hw, dy):
        w = hw[self.index_map]
        dx = torch.matmul(dy, w.t()) * self.f
        dw = torch.matmul(x.t(), dy)
        dhw = torch.zeros(self.H, dtype=dw.dtype).index_add_(0, self.flat_index, dw.reshape(-1)) * self.f
        return dx, dhw

    def step(self, x, hw, dy):
        y = self.forward(x, hw)
        dx, dhw = self.backward(x, hw, dy)
        return y, dx, dhw


def time_cpu_path(M, K, N, H, BK, BN, R, budget_s=15.0, min_reps=2, max_reps=50, seed=0):
    """Median seconds per fwd+bwd step of the CPU path within a time budget."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((M, K), generator=g)
    hw = (torch.rand((H,), generator=g) * 2 - 1) / K ** 0.5
    dy = torch.randn((M, N), generator=g)
    path = CpuPath(K, N, H, BK, BN, R)
    path.step(x, hw, dy)                       # warm-up
    times, t_end = [], time.perf_counter() + budget_s
    while len(times) < max_reps and (len(times) < min_reps or time.perf_counter() < t_end):
        t0 = time.perf_counter()
        path.step(x, hw, dy)
        times.append(time.perf_counter() - t0)
    times.sort()
    return times[len(times) // 2], len(times)
