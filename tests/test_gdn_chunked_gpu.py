"""GPU parity of the chunked (C = 64) GatedDeltaNet prefill against the sequential CPU oracle.
Tolerance (BASELINE north star): final state and outputs within 2e-3 relative of the sequential reference."""
import numpy as np
import pytest
import torch

from oracle import gdn_oracle as O
from tests import chunk_pack as P
from tests.util import *  # noqa: F401,F403

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def qt():
    import qwen_tailor_amd as q
    q._lib.lib()
    return q


def gdn_inputs(seed, T, state_scale=0.02):
    """q, k (normalized), v, a, b as BASELINE config 0 draws them, plus layer parameters and an initial state"""
    gen = torch.Generator().manual_seed(seed)
    cw, A_log, dtb, gw = layer_params(seed)
    q, k = O.normalize_qk(rand_bf(gen, (T, 16, 128)), rand_bf(gen, (T, 16, 128)))
    v, a, b = rand_bf(gen, (T, 16, 128)), rand_bf(gen, (T, 16)), rand_bf(gen, (T, 16))
    S0 = (torch.randn((16, 128, 128), generator=gen) * state_scale).numpy()
    return q, k, v, a, b, A_log, dtb, S0


@pytest.mark.parametrize("T", [64, 5, 100, 256])
def test_phase_b_on_reference_records(qt, dev, T):
    """phase B alone, fed with records packed on the CPU from the float64 chunk matrices"""
    q, k, v, a, b, A_log, dtb, S0 = gdn_inputs(40 + T, T)
    lg = O.log_decay(a, A_log, dtb)
    _, beta = O.gates(a, b, A_log, dtb)
    raw, ops, U, gC = P.chunk_records(q, k, v, lg, beta)
    y, s1 = qt.gdn_nax.phase_b(to_dev(q, dev, BF16), None, None, to_dev(ops.reshape(-1), dev), to_dev(U.reshape(-1), dev),
                               to_dev(gC.reshape(-1), dev), to_dev(S0[None], dev))
    oy, os_ = O.gated_delta_update(q[None], k[None], v[None], a[None], b[None], A_log, dtb, S0[None])
    check_rel("final state rel-L2", to_np(s1), os_, 2e-3, rel_l2)
    check_rel("final state max", to_np(s1), os_, 2e-3, rel_max)
    check_rel("y rel-L2", to_np(y), oy[0], 2e-3, rel_l2)
