"""Seeded sweeps over shapes and options of the two scans, against the same oracles and tolerances as the
hand-picked grids (tests/test_mamba1_gpu.py, tests/test_ssd_gpu.py): ragged lengths, odd channel counts per
group, state sizes off the tile sizes, optional arguments on and off in combination, packed sequences."""
import random

import pytest
import torch

from tests.test_mamba1_gpu import _run_case
from tests.test_ssd_gpu import _bwd_case

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", range(16))
def test_mamba1_random_config(seed):
    rng = random.Random(1000 + seed)
    groups = rng.choice([0, 1, 1, 2, 3])
    per = rng.choice([1, 2, 5, 8, 11, 32, 40])
    itype = rng.choice([torch.float32, torch.bfloat16, torch.float16])
    opts = dict(has_z=rng.random() < 0.7, has_D=rng.random() < 0.7, has_bias=rng.random() < 0.7,
                softplus=rng.random() < 0.7, seed=seed, var_B=rng.random() < 0.8, var_C=rng.random() < 0.8)
    if not (opts["var_B"] and opts["var_C"]) and groups == 0:
        groups = 1
    _run_case(rng.choice([1, 2, 3]), per * max(groups, 1), rng.choice([1, 3, 8, 16, 16, 24, 64]), rng.randint(1, 1500),
              itype, groups, **opts)


@pytest.mark.parametrize("seed", range(16))
def test_ssd_random_config(seed):
    rng = random.Random(2000 + seed)
    G = rng.choice([1, 1, 2, 4])
    H = G * rng.choice([1, 2, 3])
    batch, seqlen = rng.choice([1, 2]), rng.randint(17, 600)
    opts = dict(has_init=rng.random() < 0.5, has_z=rng.random() < 0.7, has_D=rng.random() < 0.7,
                with_dfinal=rng.random() < 0.5, seed=seed)
    if opts["has_D"] and rng.random() < 0.3:
        opts["D_has_hdim"] = True
    if batch == 1 and rng.random() < 0.4:
        cuts = sorted(rng.sample(range(1, seqlen), rng.randint(2, 5) - 1))
        opts["seq_lens"] = [b - a for a, b in zip([0] + cuts, cuts + [seqlen])]
    _bwd_case(batch, seqlen, H, rng.choice([16, 32, 48, 64, 96, 128]), rng.choice([8, 16, 24, 32, 64, 96, 128]), G,
              rng.choice([16, 32, 64, 128, 256]), rng.choice([torch.float32, torch.bfloat16]), **opts)
