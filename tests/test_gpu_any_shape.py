"""Shapes beyond the tuned kernels (needs an MI355X): columns longer than 1280 rows, more than 64 B
words per group, wide groups whose A columns do not fit on chip.  The reference's CPU path takes
any nrows, nwa and nwb (jni/src/BIDMach_CPUMACH.c:37,206,212), so the single-table fp32 operators
do: same bars as everywhere, 1e-4 absolute on collision-free updates, 1e-5 relative on the forward
sums, through the C ABI."""
import numpy as np
import pytest

from tests import test_gpu_parity as parity

pytestmark = pytest.mark.gpu

gpu = parity.gpu


@pytest.mark.parametrize("vexp", [0.0, 0.5])
@pytest.mark.parametrize("d,skip,ncentres", [(2048, 5, 40), (1281, 3, 60), (3000, 2, 30),
                                             (1500, 40, 12)])
def test_pos_update_long_columns(gpu, oracle, vexp, d, skip, ncentres):
    parity.test_pos_update_matches_oracle(gpu, oracle, vexp, d, skip, ncentres)


@pytest.mark.parametrize("vexp", [0.0, 0.5])
@pytest.mark.parametrize("d,nwa,nwb,G", [(2048, 5, 5, 60),     # long columns
                                         (1500, 15, 10, 30),
                                         (100, 5, 70, 40),     # more than 64 B words
                                         (300, 3, 100, 20),
                                         (1280, 40, 12, 20),   # wide group beyond LDS
                                         (2500, 20, 80, 6)])   # everything at once
def test_neg_update_any_shape(gpu, oracle, vexp, d, nwa, nwb, G):
    parity.test_neg_update_matches_oracle(gpu, oracle, vexp, d, nwa, nwb, G)


@pytest.mark.parametrize("d,skip", [(2048, 5), (1300, 12)])
def test_eval_pos_long_columns(gpu, oracle, d, skip):
    parity.test_eval_pos_matches_oracle(gpu, oracle, d, 3000, 600, skip)


@pytest.mark.parametrize("d,nwa,nwb", [(2048, 5, 5), (100, 5, 70), (1500, 15, 90)])
def test_eval_neg_any_shape(gpu, oracle, d, nwa, nwb):
    parity.test_eval_neg_matches_oracle(gpu, oracle, d, 3000, 60, nwa, nwb)


def test_neg_filt_long_columns(gpu, oracle):
    parity.test_neg_filt_matches_oracle(gpu, oracle, 1400, 5, 5)


def test_a_group_too_large_for_the_any_shape_kernel_is_rejected(gpu):
    torch, CUMACH = gpu
    d, nwa, nwb, G, V = 64, 200, 100, 2, 1000     # 200 * (100 + 256) floats of LDS
    A = torch.zeros(V, d, device="cuda")
    B = torch.zeros(V, d, device="cuda")
    WA = torch.zeros(G * nwa, dtype=torch.int32, device="cuda")
    WB = torch.zeros(G * nwb, dtype=torch.int32, device="cuda")
    assert CUMACH.word2vecNeg(d, G, nwa, nwb, WA, WB, A, B, 0.01, 0.0) == 1
