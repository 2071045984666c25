"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch

from backpack_amd import kquant, synth


def dev(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def make_weight(type_, N, K, seed):
    raw = synth.make_raw(type_, N, K, seed)
    packed = synth.pack_rows(type_, raw, N, K)
    return raw, packed, kquant.upload(type_, packed, N, K)


def check_matmul(kqo, type_, got, X, packed, N, K, bias=None, rtol=1e-3, label="", slack=1e-6):
    """The three criteria every matmul parity test applies.

    A. |got - cpu| <= atol + rtol*|cpu| with rtol as stated by the workload
       (1e-3 fp32, 1e-2 bf16 matrix cores) and atol = rtol * rms(cpu): the
       elementwise relative error is undefined where an output crosses zero, so
       the floor is one rtol of the output's rms.
    B. max |got - f64| <= 2 * max |cpu - f64| + slack*rms: the GPU result is about
       as close to the exact contraction as the CPU path it replaces (only for
       rtol <= 1e-3, i.e. fp32 accumulation of fp32 operands).  slack is 1e-6
       for VALU kernels and 1e-5 for the matrix-core row kernel, whose 4x4x4
       MFMA adds its four products and the accumulator with about 2^-19
       relative alignment loss (measured) instead of fp32 rounding.
    Returns the measured figures for reporting.
    """
    got = np.asarray(got, dtype=np.float32).reshape(-1, N)
    cpu = kqo.matmul(type_, X, packed, N, K, bias=bias)
    f64 = kqo.matmul_f64(type_, X, packed, N, K, bias=bias)
    rms = float(np.sqrt(np.mean(f64 ** 2))) + 1e-30
    err = np.abs(got.astype(np.float64) - cpu)
    tol = rtol * rms + rtol * np.abs(cpu)
    worst = float((err / tol).max())
    assert worst <= 1.0, f"{label}: criterion A violated, err/tol={worst:.3g}"
    e_gpu = float(np.abs(got - f64).max())
    e_cpu = float(np.abs(cpu - f64).max())
    if rtol <= 1e-3:
        assert e_gpu <= 2 * e_cpu + slack * rms, f"{label}: GPU error {e_gpu:.3g} vs CPU error {e_cpu:.3g}"
    return dict(max_rel=float((err / (np.abs(cpu) + rtol * rms)).max()), e_gpu=e_gpu, e_cpu=e_cpu, rms=rms)
