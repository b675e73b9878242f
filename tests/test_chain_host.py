"""The library's templates, compiled for the host cores, against the oracle.

Runs without a GPU: it exercises Variable, the operation nodes, the op logic of
the benchmark graph and run() exactly as the kernels do, through the host entry
points of the C ABI.
"""
import numpy as np

from tests._metrics import abs_or_rel, chain_closed_form, chain_inputs, covariance_condition
from xyz_autodiff_cuda_amd import chain


def test_fp64_templates_match_oracle_and_closed_form(oracle, xad):
    inputs = chain_inputs(50000, seed=21)
    got = np.stack(chain.host_forward_backward(inputs, np.float64, num_threads=4))
    assert abs_or_rel(got, oracle.chain_soa(inputs, np.float64)).max() < 1e-10
    assert abs_or_rel(got, chain_closed_form(inputs)[0]).max() < 1e-9


def test_fp32_templates_match_oracle(oracle, xad):
    inputs = chain_inputs(200000, seed=22)
    got = np.stack(chain.host_forward_backward(inputs, np.float32, num_threads=4))
    ref32 = oracle.chain_soa(inputs, np.float32)
    ref64 = oracle.chain_soa(inputs, np.float64)
    kappa = covariance_condition(inputs[0], inputs[1])
    for ref in (ref32, ref64):
        e = abs_or_rel(got, ref)
        assert e[0].max() < 1e-5  # forward value: 1e-5 on every problem
        assert e[:, kappa <= 7.4].max(initial=0.0) < 1e-5  # gradients, well-conditioned Sigma
        assert (e / np.maximum(1.0, kappa)).max() < 1e-5  # gradients, scaled by cond(Sigma)
    # and never less accurate than the reference formulation is in fp32
    assert abs_or_rel(got, ref64).max() <= 2.0 * abs_or_rel(ref32, ref64).max()


def test_thread_count_does_not_change_results(xad):
    inputs = chain_inputs(10001, seed=23)
    a = np.stack(chain.host_forward_backward(inputs, np.float32, num_threads=1))
    b = np.stack(chain.host_forward_backward(inputs, np.float32, num_threads=7))
    assert np.array_equal(a, b)


def test_empty_input(xad):
    outs = chain.host_forward_backward([np.zeros(0, np.float32)] * 6)
    assert all(o.size == 0 for o in outs)
