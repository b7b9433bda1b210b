"""Writes tests/golden/vectors.npz: tiny known-answer cases of the three operators.

The expected values do not come from the oracle or from the HIP kernels: every output is computed
here by explicit Python loops over positions, channels and states in float64 numpy, straight from
the recurrences (reference mamba_ssm/ops/selective_scan_interface.py:142-193,
mamba_ssm/ops/triton/selective_state_update.py:224-285, mamba_ssm/ops/triton/ssd_combined.py:728-775
for the meaning of the SSD arguments), and the Mamba-1 gradients by central differences of that
loop.  They are regression vectors of this repository, not outputs of the reference.

    python tests/golden/make_vectors.py
"""
import os

import numpy as np


def softplus(x):
    return np.where(x <= 20.0, np.log1p(np.exp(np.minimum(x, 20.0))), x)


def silu(x):
    return x / (1.0 + np.exp(-x))


def scan_loop(u, delta, A, B, C, D, z, delta_bias):
    """u, delta, z: (b, d, L); A: (d, n); B, C: (b, g, n, L); D, delta_bias: (d,).  softplus on."""
    b, d, L = u.shape
    g, n = B.shape[1], B.shape[2]
    out = np.zeros((b, d, L))
    last = np.zeros((b, d, n))
    for ib in range(b):
        for ch in range(d):
            grp = ch // (d // g)
            h = np.zeros(n)
            for t in range(L):
                dl = softplus(delta[ib, ch, t] + delta_bias[ch])
                y = 0.0
                for s in range(n):
                    h[s] = np.exp(dl * A[ch, s]) * h[s] + dl * B[ib, grp, s, t] * u[ib, ch, t]
                    y += C[ib, grp, s, t] * h[s]
                out[ib, ch, t] = (y + D[ch] * u[ib, ch, t]) * silu(z[ib, ch, t])
            last[ib, ch] = h
    return out, last


def ssd_loop(x, dt, A, B, C, D, z, dt_bias, init, seq_idx):
    """x, z: (b, L, h, p); dt: (b, L, h); A, D, dt_bias: (h,); B, C: (b, L, g, n); init: (b, h, p, n)."""
    b, L, H, P = x.shape
    g, n = B.shape[2], B.shape[3]
    out = np.zeros((b, L, H, P))
    fin = np.zeros((b, H, P, n))
    for ib in range(b):
        for hd in range(H):
            grp = hd // (H // g)
            st = init[ib, hd].copy()
            prev = 0
            for t in range(L):
                if seq_idx[ib, t] != prev:
                    st[:] = 0.0
                prev = seq_idx[ib, t]
                step = softplus(dt[ib, t, hd] + dt_bias[hd])
                for pp in range(P):
                    y = 0.0
                    for s in range(n):
                        st[pp, s] = np.exp(step * A[hd]) * st[pp, s] + step * x[ib, t, hd, pp] * B[ib, t, grp, s]
                        y += st[pp, s] * C[ib, t, grp, s]
                    out[ib, t, hd, pp] = (y + D[hd] * x[ib, t, hd, pp]) * silu(z[ib, t, hd, pp])
            fin[ib, hd] = st
    return out, fin


def step_loop(state, x, dt, A, B, C, D, z, dt_bias):
    """state: (b, h, p, n); x, z, dt, dt_bias-expanded: (b, h, p); A: (h, p, n); B, C: (b, g, n); D: (h, p)."""
    b, H, P, n = state.shape
    g = B.shape[1]
    new = state.copy()
    out = np.zeros((b, H, P))
    for ib in range(b):
        for hd in range(H):
            grp = hd // (H // g)
            for pp in range(P):
                step = softplus(dt[ib, hd, pp] + dt_bias[hd, pp])
                y = 0.0
                for s in range(n):
                    new[ib, hd, pp, s] = state[ib, hd, pp, s] * np.exp(step * A[hd, pp, s]) + step * B[ib, grp, s] * x[ib, hd, pp]
                    y += new[ib, hd, pp, s] * C[ib, grp, s]
                out[ib, hd, pp] = (y + D[hd, pp] * x[ib, hd, pp]) * silu(z[ib, hd, pp])
    return new, out


def main():
    rng = np.random.default_rng(20240607)
    v = {}
    # Mamba-1: batch 2, 4 channels in 2 groups, 19 positions, 3 states; gradients of sum(out * dout)
    b, d, L, n, g = 2, 4, 19, 3, 2
    m = dict(u=rng.standard_normal((b, d, L)), delta=rng.standard_normal((b, d, L)) - 1.0,
             A=-rng.uniform(0.2, 1.5, (d, n)), B=rng.standard_normal((b, g, n, L)), C=rng.standard_normal((b, g, n, L)),
             D=rng.standard_normal(d), z=rng.standard_normal((b, d, L)), delta_bias=rng.standard_normal(d) * 0.5)
    dout = rng.standard_normal((b, d, L))
    out, last = scan_loop(**m)
    for k, a in m.items():
        v["m1_" + k] = a
    v.update(m1_dout=dout, m1_out=out, m1_last_state=last)
    eps = 1e-6
    for k, a in m.items():
        grad = np.zeros_like(a)
        it = np.nditer(a, flags=["multi_index"])
        for _ in it:
            idx = it.multi_index
            keep = a[idx]
            a[idx] = keep + eps
            hi = (scan_loop(**m)[0] * dout).sum()
            a[idx] = keep - eps
            lo = (scan_loop(**m)[0] * dout).sum()
            a[idx] = keep
            grad[idx] = (hi - lo) / (2 * eps)
        v["m1_d" + k] = grad
    # SSD: batch 1 packing three sequences (ids 0, 1, 2), 2 heads, headdim 3, 4 states, initial state
    b, L, H, P, n, g = 1, 21, 2, 3, 4, 1
    s = dict(x=rng.standard_normal((b, L, H, P)), dt=rng.standard_normal((b, L, H)) - 1.0, A=-rng.uniform(0.5, 2.0, H),
             B=rng.standard_normal((b, L, g, n)), C=rng.standard_normal((b, L, g, n)), D=rng.uniform(0, 1, H),
             z=rng.standard_normal((b, L, H, P)), dt_bias=rng.standard_normal(H) * 0.3,
             init=rng.standard_normal((b, H, P, n)) * 0.1,
             seq_idx=np.concatenate([np.zeros(8), np.ones(6), np.full(7, 2)]).astype(np.int32)[None])
    out, fin = ssd_loop(**s)
    for k, a in s.items():
        v["ssd_" + k] = a
    v.update(ssd_out=out, ssd_final_states=fin)
    # decode step: batch 2, 2 heads, headdim 3, 5 states (not a multiple of 4), per-element A
    b, H, P, n, g = 2, 2, 3, 5, 1
    q = dict(state=rng.standard_normal((b, H, P, n)) * 0.1, x=rng.standard_normal((b, H, P)),
             dt=rng.standard_normal((b, H, P)) - 1.0, A=-rng.uniform(0.5, 2.0, (H, P, n)), B=rng.standard_normal((b, g, n)),
             C=rng.standard_normal((b, g, n)), D=rng.uniform(0, 1, (H, P)), z=rng.standard_normal((b, H, P)),
             dt_bias=rng.standard_normal((H, P)) * 0.3)
    new, out = step_loop(**q)
    for k, a in q.items():
        v["step_" + k] = a
    v.update(step_new_state=new, step_out=out)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vectors.npz")
    np.savez_compressed(path, **v)
    print(path, sum(a.size for a in v.values()), "values")


if __name__ == "__main__":
    main()
