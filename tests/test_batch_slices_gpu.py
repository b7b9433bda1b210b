"""Batches beyond what one launch's grid can index (65535 batch rows of the Mamba-1 scan, 65535 (batch, head) pairs
of the SSD scan) are served in slices of batch rows inside the C entry points.  One call over such a batch must equal
the same operator called on two halves that each fit one launch: outputs, last / final states and every gradient."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_mamba1_more_than_65535_batch_rows():
    from mamba_amd.ops.selective_scan_interface import selective_scan_fn
    batch, dim, L, N = 65535 + 700, 4, 24, 4
    g = torch.Generator(device="cuda").manual_seed(0)
    rn = lambda *s: torch.randn(*s, device="cuda", generator=g)
    t = dict(u=rn(batch, dim, L), delta=0.5 * torch.rand(batch, dim, L, device="cuda", generator=g), A=-torch.rand(dim, N, device="cuda", generator=g),
             B=rn(batch, 1, N, L), C=rn(batch, 1, N, L), D=rn(dim), z=rn(batch, dim, L), delta_bias=rn(dim) - 2)
    dout = rn(batch, dim, L)
    names = list(t)

    def run(rows):
        x = {k: (t[k][rows] if t[k].dim() >= 3 else t[k]).clone().requires_grad_() for k in names}
        out, last = selective_scan_fn(*[x[k] for k in names], delta_softplus=True, return_last_state=True)
        out.backward(dout[rows])
        return out, last, x

    out, last, x = run(slice(0, batch))
    half = batch // 2
    parts = [run(slice(0, half)), run(slice(half, batch))]
    assert torch.equal(out, torch.cat([p[0] for p in parts])) and torch.equal(last, torch.cat([p[1] for p in parts]))
    for k in ("u", "delta", "z", "B", "C"):
        assert torch.equal(x[k].grad, torch.cat([p[2][k].grad for p in parts])), k
    for k in ("A", "D", "delta_bias"):   # sums over the batch: the halves add up (another order of the same fp32 terms)
        want = parts[0][2][k].grad + parts[1][2][k].grad
        assert torch.allclose(x[k].grad, want, rtol=1e-4, atol=1e-3), k


def test_ssd_more_than_65535_batch_head_pairs():
    from mamba_amd.ops.triton.ssd_combined import mamba_chunk_scan_combined
    batch, L, H, P, N, G, Q = 16384 + 300, 64, 4, 32, 16, 2, 32
    g = torch.Generator(device="cuda").manual_seed(1)
    rn = lambda *s: torch.randn(*s, device="cuda", generator=g)
    t = dict(x=rn(batch, L, H, P), dt=rn(batch, L, H), A=-torch.rand(H, device="cuda", generator=g) - 1, B=rn(batch, L, G, N),
             C=rn(batch, L, G, N), D=rn(H), z=rn(batch, L, H, P), dt_bias=rn(H) - 3, initial_states=0.1 * rn(batch, H, P, N))
    dout, dfin = rn(batch, L, H, P), rn(batch, H, P, N)
    names = list(t)

    def run(rows):
        x = {k: (t[k][rows] if t[k].dim() >= 3 else t[k]).clone().requires_grad_() for k in names}
        out, fin = mamba_chunk_scan_combined(x["x"], x["dt"], x["A"], x["B"], x["C"], Q, D=x["D"], z=x["z"], dt_bias=x["dt_bias"],
                                             initial_states=x["initial_states"], dt_softplus=True, return_final_states=True)
        (out * dout[rows]).sum().add((fin * dfin[rows]).sum()).backward()
        return out, fin, x

    out, fin, x = run(slice(0, batch))
    half = batch // 2
    parts = [run(slice(0, half)), run(slice(half, batch))]
    assert torch.equal(out, torch.cat([p[0] for p in parts])) and torch.equal(fin, torch.cat([p[1] for p in parts]))
    for k in ("x", "z", "dt", "B", "C", "initial_states"):   # dB / dC / ddt add with float atomics: a few ulps apart
        want = torch.cat([p[2][k].grad for p in parts])
        assert torch.allclose(x[k].grad, want, rtol=1e-4, atol=1e-4), k
    for k in ("A", "D", "dt_bias"):
        want = parts[0][2][k].grad + parts[1][2][k].grad
        assert torch.allclose(x[k].grad, want, rtol=1e-3, atol=float(want.abs().max()) * 1e-4), k
