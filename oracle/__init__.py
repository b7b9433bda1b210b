"""CPU oracle for the Mamba scan hot path.

TEST INFRASTRUCTURE ONLY.  Nothing under mamba_amd/ imports this package; it is used by
tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline leg as the checker and
the timed CPU baseline, never as a compute path of the product.

Each function restates, in plain PyTorch on the CPU, the algorithm of one of the reference's
own pure-PyTorch reference functions (cited per function).  tests/test_oracle_*.py pin the
restatements against closed forms, library routines, brute force and torch.autograd.gradcheck.
"""
