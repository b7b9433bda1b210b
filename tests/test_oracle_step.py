"""Pins the decode-step oracle (oracle/step.py): T steps == a length-T scan of the Mamba-1 oracle, one
step by hand, head/group broadcasting and the batch-index gather."""
import torch
import torch.nn.functional as F

from oracle.mamba1 import selective_scan_oracle
from oracle.step import selective_state_update_oracle

f64 = torch.float64


def test_steps_equal_scan():
    g = torch.Generator().manual_seed(0)
    b, d, n, T = 2, 5, 4, 17
    u, delta, z = (torch.randn(b, d, T, generator=g, dtype=f64) for _ in range(3))
    A = -torch.rand(d, n, generator=g, dtype=f64) - 0.3
    B, C = torch.randn(b, n, T, generator=g, dtype=f64), torch.randn(b, n, T, generator=g, dtype=f64)
    D, bias = torch.randn(d, generator=g, dtype=f64), torch.randn(d, generator=g, dtype=f64)
    y, last = selective_scan_oracle(u, delta, A, B, C, D, z, bias, True, True, compute_dtype=f64)
    state = torch.zeros(b, d, n, dtype=f64)
    ys = [selective_state_update_oracle(state, u[:, :, t], delta[:, :, t], A, B[:, :, t], C[:, :, t], D=D,
                                        z=z[:, :, t], dt_bias=bias, dt_softplus=True, compute_dtype=f64)
          for t in range(T)]
    assert torch.allclose(torch.stack(ys, 2), y, atol=1e-12) and torch.allclose(state, last, atol=1e-12)


def test_one_step_by_hand_with_heads_and_groups():
    g = torch.Generator().manual_seed(1)
    b, H, P, n, G = 2, 4, 3, 2, 2
    state = torch.randn(b, H, P, n, generator=g, dtype=f64)
    x, dt, z = (torch.randn(b, H, P, generator=g, dtype=f64) for _ in range(3))
    A = -torch.rand(H, P, n, generator=g, dtype=f64)
    B, C = torch.randn(b, G, n, generator=g, dtype=f64), torch.randn(b, G, n, generator=g, dtype=f64)
    D, bias = torch.randn(H, P, generator=g, dtype=f64), torch.randn(H, P, generator=g, dtype=f64)
    s0 = state.clone()
    out = selective_state_update_oracle(state, x, dt, A, B, C, D=D, z=z, dt_bias=bias, dt_softplus=True,
                                        compute_dtype=f64)
    for bi in range(b):
        for h in range(H):
            gi = h // (H // G)
            for p in range(P):
                d = F.softplus(dt[bi, h, p] + bias[h, p])
                acc = 0.0
                for k in range(n):
                    new = s0[bi, h, p, k] * torch.exp(d * A[h, p, k]) + d * B[bi, gi, k] * x[bi, h, p]
                    assert torch.allclose(state[bi, h, p, k], new, atol=1e-12)
                    acc = acc + new * C[bi, gi, k]
                acc = (acc + D[h, p] * x[bi, h, p]) * z[bi, h, p] * torch.sigmoid(z[bi, h, p])
                assert torch.allclose(out[bi, h, p], acc, atol=1e-12)


def test_batch_indices_and_padding():
    g = torch.Generator().manual_seed(2)
    state = torch.randn(5, 3, 2, generator=g, dtype=f64)
    x, dt = torch.randn(3, 3, generator=g, dtype=f64), torch.rand(3, 3, generator=g, dtype=f64)
    A = -torch.rand(3, 2, generator=g, dtype=f64)
    B, C = torch.randn(3, 2, generator=g, dtype=f64), torch.randn(3, 2, generator=g, dtype=f64)
    idx = torch.tensor([4, -1, 0], dtype=torch.int32)
    s0 = state.clone()
    out = selective_state_update_oracle(state, x, dt, A, B, C, state_batch_indices=idx, compute_dtype=f64)
    ref_state = s0.clone()
    dense = ref_state[[4, 0]]
    o = selective_state_update_oracle(dense, x[[0, 2]], dt[[0, 2]], A, B[[0, 2]], C[[0, 2]], compute_dtype=f64)
    assert torch.allclose(out[[0, 2]], o) and float(out[1].abs().max()) == 0.0
    assert torch.allclose(state[[4, 0]], dense) and torch.equal(state[[1, 2, 3]], s0[[1, 2, 3]])
