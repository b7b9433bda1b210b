"""The measurement yardsticks of the library move exactly the bytes they say they do: the row pass writes the xor / sum
of its inputs to every row, and reports the bytes of the launch."""
import ctypes

import pytest
import torch

from mamba_amd import _lib

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n_in", [2, 4])
def test_row_pass_touches_every_row_once(n_in):
    torch.manual_seed(n_in)
    batch, seqlen, nheads = 2, 512, 12
    shape = (batch, seqlen, nheads, 32)   # 64 16-bit values per row, seen as 32 int32
    ins = [torch.randint(-2**31, 2**31 - 1, shape, dtype=torch.int32, device="cuda") for _ in range(n_in)]
    outs = [torch.zeros(shape, dtype=torch.int32, device="cuda") for _ in range(2)]
    pin = (ctypes.c_void_p * n_in)(*[t.data_ptr() for t in ins])
    pout = (ctypes.c_void_p * 2)(*[t.data_ptr() for t in outs])
    lib = _lib.load()
    moved = lib.mamba_hip_rows_probe(pin, n_in, pout, batch, seqlen, nheads, _lib.current_stream(ins[0].device))
    torch.cuda.synchronize()
    assert moved == (n_in + 2) * batch * seqlen * nheads * 128
    if n_in == 2:
        assert torch.equal(outs[0], ins[0]) and torch.equal(outs[1], ins[1])
    else:
        assert torch.equal(outs[0], ins[0] ^ ins[1])
        assert torch.equal(outs[1], ins[3] + ins[2])   # int32 addition wraps, as the kernel's does


def test_row_pass_rejects_what_it_cannot_index():
    lib = _lib.load()
    t = torch.zeros(1, 256, 2, 32, dtype=torch.int32, device="cuda")
    pin = (ctypes.c_void_p * 2)(t.data_ptr(), t.data_ptr())
    pout = (ctypes.c_void_p * 2)(t.data_ptr(), t.data_ptr())
    s = _lib.current_stream(t.device)
    assert lib.mamba_hip_rows_probe(pin, 3, pout, 1, 256, 2, s) < 0      # two or four inputs
    assert lib.mamba_hip_rows_probe(pin, 2, pout, 1, 200, 2, s) < 0      # whole chunks of 256 positions
    assert lib.mamba_hip_rows_probe(None, 2, pout, 1, 256, 2, s) < 0
