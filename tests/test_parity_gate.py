"""The parity gates themselves: wrong results must fail them.  CPU only: the "device output" here is the oracle fed
with deliberately wrong inputs, on the headline workload (config 3), where outputs are small (|out| ~ 0.015) and the
tolerance the task states (2e-2 max-abs) is larger than the signal."""
import numpy as np
import pytest
import torch

from helpers import TOL, assert_close, np64, oracle_fused


@pytest.fixture(scope="module")
def c3(oracle):
    from inference_lib_amd import cases
    c = cases.baseline_case(3)
    out, lse, _ = oracle_fused(oracle, c)
    return c, out, lse


def _as_device_output(a, dtype=torch.bfloat16):
    return torch.from_numpy(np.asarray(a)).to(dtype)


def test_gate_accepts_the_oracle_rounded_to_storage(c3):
    c, out, lse = c3
    assert_close("out", _as_device_output(out), out, TOL[c.dtype])
    assert_close("lse", _as_device_output(lse, torch.float32), lse, TOL[c.dtype])


def test_out_gate_alone_rejects_a_dropped_fragment(oracle, c3):
    """One fragment (the 110 newest tokens of worker 2, of 12 528 visible ones) missing from the attention: the output
    gate must notice without the help of the LSE gate.  The stated 2e-2 bound alone does not."""
    c, out, lse = c3
    assert c.lens[7] == 110
    keep = [f for f in range(c.F) if f != 7]
    wrong, _, _ = oracle.fused_reference(
        np64(c.q), c.locations.numpy()[keep], [np64(c.keys[f]) for f in keep], [np64(c.values[f]) for f in keep], c.scale,
        np64(c.cos)[keep], np64(c.sin)[keep], storage=c.dtype)
    err = np.abs(wrong - out).max()
    assert err < float(TOL[c.dtype]), "the stated bound would have let this through"
    with pytest.raises(AssertionError):
        assert_close("out", _as_device_output(wrong), out, TOL[c.dtype])


def test_out_gate_rejects_zeros_and_a_wrong_scale(c3):
    c, out, lse = c3
    with pytest.raises(AssertionError):
        assert_close("out", torch.zeros(out.shape, dtype=torch.bfloat16), out, TOL[c.dtype])
    with pytest.raises(AssertionError):
        assert_close("out", _as_device_output(out * 1.1), out, TOL[c.dtype])


def test_lse_gate_rejects_a_dropped_tile(c3):
    """32 of 12 528 keys missing changes the LSE by ~2.5e-3: caught by the 2e-3 LSE bound, not by the stated 2e-2."""
    c, out, lse = c3
    wrong = lse + np.log1p(-32.0 / 12528.0)
    with pytest.raises(AssertionError):
        assert_close("lse", _as_device_output(wrong, torch.float32), lse, TOL[c.dtype])
