"""Shared helpers of the parity tests: run a Case through the C ABI and through the oracle."""
import numpy as np
import torch

class Tol(float):
    """A parity bound.  The float value is the bound the task states (max-abs against the fp32/fp64 oracle: bf16 / fp16
    2e-2, fp32 1e-4).  For the 16-bit types that alone is weak where outputs are small (a softmax over 12 000 keys of
    N(0,1) values gives |out| ~ 0.015), so assert_close also applies a bound relative to the signal:
        out: max|d| <= rel * max|reference| + floor        lse: max|d| <= lse
    and passes only if both hold."""

    def __new__(cls, stated, rel=None, floor=0.0, lse=None):
        t = super().__new__(cls, stated)
        t.rel, t.floor, t.lse = rel, floor, lse
        return t

    def out_bound(self, want: np.ndarray) -> float:
        if self.rel is None:
            return float(self)
        fin = np.isfinite(want)
        peak = float(np.abs(want[fin]).max()) if fin.any() else 0.0
        return min(float(self), self.rel * peak + self.floor)

    def lse_bound(self) -> float:
        return float(self) if self.lse is None else min(float(self), self.lse)


TOL = {"f32": Tol(1e-4), "f16": Tol(2e-2, rel=2.0 ** -7, floor=1e-3, lse=2e-3), "bf16": Tol(2e-2, rel=2.0 ** -7, floor=1e-3, lse=2e-3)}


def np64(t: torch.Tensor) -> np.ndarray:
    return t.detach().to("cpu").to(torch.float64).numpy()


def oracle_fused(oracle, case, second_half_index="first"):
    out, lse, rq = oracle.fused_reference(
        np64(case.q), case.locations.cpu().numpy(), [np64(k) for k in case.keys], [np64(v) for v in case.values],
        case.scale, np64(case.cos), np64(case.sin), storage=case.dtype, second_half_index=second_half_index)
    return out, lse, rq


def run_fused(case_dev, *, splits=0, with_rq=True, with_lse=True, row_blocks=0):
    """Call hw_fused_attention through the C ABI on a Case whose tensors are on the GPU."""
    from inference_lib_amd import _lib
    dev = case_dev.q.device
    W, Hq, S, E = case_dev.q.shape
    out = torch.full((W, Hq, S, E), float("nan"), dtype=case_dev.q.dtype, device=dev)
    lse = torch.full((W, Hq, S), float("nan"), dtype=torch.float32, device=dev) if with_lse else None
    rq = torch.full((case_dev.F, W, Hq, S, E), float("nan"), dtype=case_dev.q.dtype, device=dev) if with_rq else None
    pr = _lib.Problem(q=case_dev.q, locations=case_dev.locations, keys=case_dev.keys, values=case_dev.values,
                      scale=case_dev.scale, out=out, cosines=case_dev.cos, sines=case_dev.sin, rq=rq, lse=lse, splits=splits,
                      row_blocks=row_blocks)
    pr.run()
    torch.cuda.synchronize()
    return out, lse, rq


def assert_close(name, got: torch.Tensor, want: np.ndarray, tol: float):
    """max-abs comparison; a Tol also brings the signal-relative bound (names containing "lse" use its lse bound)."""
    if isinstance(tol, Tol):
        tol = tol.lse_bound() if "lse" in name else tol.out_bound(np.asarray(want, dtype=np.float64))
    g = np64(got)
    assert g.shape == want.shape, (name, g.shape, want.shape)
    assert np.isfinite(g[np.isfinite(want)]).all(), f"{name}: non-finite values"
    both = np.isfinite(want)
    err = float(np.abs(g[both] - want[both]).max()) if both.any() else 0.0
    assert err <= tol, f"{name}: max abs err {err:.3e} > {tol:.1e}"
    # -inf entries (empty rows) must match exactly
    assert (np.isneginf(g) == np.isneginf(want)).all(), f"{name}: -inf pattern differs"
    return err
