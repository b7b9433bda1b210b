"""The fused SSD kernels (forward scan, backward dx and chunk-state dB / dC: chosen for bf16 on 16-byte aligned rows) against the tiled
kernels the same entry points fall back to: the same problem is run twice through mamba_chunk_scan_combined, once
on ordinary tensors and once on copies of x and z whose rows start 8 bytes off a 16-byte boundary, which the fused
kernels decline.  Both pipelines compute the same sums in fp32 from the same bf16 operands, so outputs and
gradients agree to the rounding of the bf16 results (the oracle comparisons of each pipeline are in
test_ssd_gpu.py and test_random_configs_gpu.py; this test pins the two against each other on shapes those draw
rarely: several heads per workgroup, groups, packed sequences, a ragged last chunk; the fused chunk-state dB / dC
kernels decline the same copies, so their sums are pinned against the tiled ones here too)."""
import pytest
import torch

from mamba_amd.ops.triton.ssd_combined import mamba_chunk_scan_combined

pytestmark = pytest.mark.gpu


def _off_alignment(t):
    """A copy of t (b, L, H, P) with the same values whose rows start 8 bytes after a 16-byte boundary."""
    b, L, H, P = t.shape
    big = torch.zeros(b, L, H, P + 8, device=t.device, dtype=t.dtype)
    view = big[..., 4:4 + P]
    view.copy_(t)
    assert view.data_ptr() % 16 == 8 and view.stride(-1) == 1
    return view


def _run(x, dt, A, B, C, D, z, dt_bias, seq_idx, chunk, dout):
    leaves = [t.detach().clone().requires_grad_(True) for t in (dt, A, B, C, D, dt_bias)]
    xl = x.detach().requires_grad_(True)          # keeps the storage (and its alignment) of what was passed in
    zl = z.detach().requires_grad_(True)
    dt_, A_, B_, C_, D_, bias_ = leaves
    out = mamba_chunk_scan_combined(xl, dt_, A_, B_, C_, chunk, D=D_, z=zl, dt_bias=bias_, dt_softplus=True, seq_idx=seq_idx)
    out.backward(dout)
    return out.detach(), [xl.grad, zl.grad] + [t.grad for t in leaves]


@pytest.mark.parametrize("batch,seqlen,nheads,headdim,ngroups,dstate,chunk,packed", [
    (2, 512, 16, 64, 1, 128, 256, False),   # 16 heads of one group in one workgroup
    (1, 700, 8, 64, 2, 64, 128, False),     # ragged last chunk, two groups
    (1, 1024, 12, 32, 3, 128, 256, True),   # packed sequences, headdim 32
    (2, 256, 4, 64, 4, 64, 64, False),      # one head per group: one head per workgroup
    (1, 384, 6, 32, 2, 64, 64, False),      # the smallest tiles of every fused kernel
    (1, 640, 4, 64, 1, 128, 128, True),     # chunk 128 with 128 states, packed
    (2, 200, 8, 32, 1, 128, 64, False),     # headdim 32 with 128 states, ragged
    (1, 512, 10, 32, 1, 64, 256, False),    # headdim 32 with 64 states, chunk 256
    (1, 900, 8, 64, 2, 64, 256, True),      # chunk 256, packed, a ragged last chunk with whole tiles past the end
    (2, 300, 4, 64, 1, 128, 256, False),    # chunk 256, second chunk of 44 positions
])
def test_fused_and_tiled_agree(batch, seqlen, nheads, headdim, ngroups, dstate, chunk, packed):
    _compare(batch, seqlen, nheads, headdim, ngroups, dstate, chunk, packed)


def test_fused_and_tiled_agree_with_a_D_per_channel():
    """D of shape (nheads, headdim): dD per channel leaves the fused dz / state-gradient kernel as column sums."""
    _compare(2, 512, 8, 64, 2, 128, 256, False, d_per_channel=True)
    _compare(1, 256, 4, 32, 1, 128, 128, False, d_per_channel=True)


def _compare(batch, seqlen, nheads, headdim, ngroups, dstate, chunk, packed, d_per_channel=False):
    torch.manual_seed(batch * 1000 + seqlen + nheads)
    dev, dt16 = "cuda", torch.bfloat16
    x = torch.randn(batch, seqlen, nheads, headdim, device=dev, dtype=dt16)
    z = torch.randn_like(x)
    dt = (torch.rand(batch, seqlen, nheads, device=dev) * 0.5).to(dt16)
    A = -(torch.rand(nheads, device=dev) + 0.5)
    B = torch.randn(batch, seqlen, ngroups, dstate, device=dev, dtype=dt16)
    C = torch.randn(batch, seqlen, ngroups, dstate, device=dev, dtype=dt16)
    D = torch.randn(nheads, headdim, device=dev) if d_per_channel else torch.randn(nheads, device=dev)
    dt_bias = torch.rand(nheads, device=dev) - 1.0
    seq_idx = None
    if packed:
        cuts = torch.tensor([c for c in (0, 130, 131, 400, 777) if c < seqlen] + [seqlen], device=dev)
        seq_idx = (torch.arange(seqlen, device=dev)[None, :] >= cuts[1:-1, None]).sum(0).to(torch.int32)[None].expand(batch, -1).contiguous()
    dout = torch.randn_like(x)

    out_f, grads_f = _run(x, dt, A, B, C, D, z, dt_bias, seq_idx, chunk, dout)
    out_t, grads_t = _run(_off_alignment(x), dt, A, B, C, D, _off_alignment(z), dt_bias, seq_idx, chunk, dout)

    def close(a, b, name):
        a, b = a.float(), b.float()
        scale = float(b.abs().max()) + 1e-6
        err = float((a - b).abs().max()) / scale
        # both sides round fp32 sums to bf16 (outputs, dx, dz, dB, dC) or add the same fp32 terms in another order
        assert err < 1.6e-2, f"{name}: fused and tiled pipelines differ by {err:.3e} of the largest value"

    close(out_f, out_t, "out")
    for name, gf, gt in zip(("dx", "dz", "ddt", "dA", "dB", "dC", "dD", "ddt_bias"), grads_f, grads_t):
        close(gf, gt, name)


@pytest.mark.parametrize("misaligned", [False, True])
def test_forward_without_gradients_skips_the_pre_gate_copy(misaligned):
    """Under torch.no_grad() the scan is not handed a buffer for the output before the gate (only the backward pass
    reads it): the gated output is bit for bit the one of a differentiated call, on the fused and on the tiled
    kernels."""
    torch.manual_seed(5)
    dev, dt16 = "cuda", torch.bfloat16
    batch, seqlen, nheads, headdim, ngroups, dstate, chunk = 2, 600, 8, 64, 2, 128, 256
    x = torch.randn(batch, seqlen, nheads, headdim, device=dev, dtype=dt16)
    z = torch.randn_like(x)
    if misaligned:
        x, z = _off_alignment(x), _off_alignment(z)
    dt = (torch.rand(batch, seqlen, nheads, device=dev) * 0.5).to(dt16)
    A = -(torch.rand(nheads, device=dev) + 0.5)
    B = torch.randn(batch, seqlen, ngroups, dstate, device=dev, dtype=dt16)
    C = torch.randn(batch, seqlen, ngroups, dstate, device=dev, dtype=dt16)
    D = torch.randn(nheads, device=dev)
    with torch.no_grad():
        plain = mamba_chunk_scan_combined(x, dt, A, B, C, chunk, D=D, z=z, dt_softplus=True)
    xg = x.detach().requires_grad_(True)
    tracked = mamba_chunk_scan_combined(xg, dt, A, B, C, chunk, D=D, z=z, dt_softplus=True)
    assert tracked.requires_grad and not plain.requires_grad
    assert torch.equal(plain, tracked.detach())
