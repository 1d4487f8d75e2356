"""Shared helpers of the parity tests: the tolerances of the task statement, one rule per arithmetic, and an error report.

fp32 (values and gradients): every element within rtol 1e-4 of the oracle, with an absolute floor of 1e-4 of the
tensor's largest magnitude (the statement names no atol; where the normaliser sum b nearly cancels, its fp32 rounding
is 1e-4 of b, and exactly those rows carry the largest |h|).

fp16 / bf16: rtol 2e-2, atol 2e-3, element by element, literally.  The split mode of the kernels (MLSTM_PRECISE) is
held to exactly that, as is every comparison of a 16-bit kernel with a CPU evaluation of the same 16-bit algorithm.
The default 16-bit kernels round the weights of a tile's second product to the element type (as the reference's CUDA
kernels do, cuda-src/mlstm_forward.cu:143-160), and an output element is a sum of terms that can be fifty times its
own size: that rounding alone puts 1-6 % of bf16 elements outside the literal bound, in a float64 CPU evaluation of
the algorithm exactly as on the GPU (tests/test_gpu_tolerance.py measures both).  For those kernels the bound gains
one term, NOISE_SIGMAS standard deviations of that rounding noise as the oracle predicts it per element
(oracle.mlstm_rounding_noise): |got - ref| <= atol + rtol |ref| + 6 sigma.  A kernel that loses precision anywhere
else, or computes something different, fails it by orders of magnitude; no test scales a tolerance or picks a seed.
Both kinds of test also bound the error's rms: REL_RMS of the reference's rms, or, where the predicted noise is larger
than that (gate regimes in which dC~ nearly cancels), 1.25 times the predicted rms.
"""
import torch

from oracle import mlstm_oracle as O

HALF_RTOL, HALF_ATOL = 2e-2, 2e-3
F32_RTOL, F32_ATOL_FRAC = 1e-4, 1e-4
NOISE_SIGMAS = 6.0
REL_RMS = {torch.float32: 1e-4, torch.float16: 1.5e-3, torch.bfloat16: 8e-3}
GRAD_NAMES = ["dq", "dk", "dv", "df", "di"]


def literal_violations(got, ref):
    """Fraction of elements outside the literal 16-bit bound, and the error's rms relative to the reference's."""
    got, ref = got.detach().cpu().double(), ref.detach().cpu().double()
    err = (got - ref).abs()
    bad = err > HALF_ATOL + HALF_RTOL * ref.abs()
    rms = float(ref.pow(2).mean().sqrt())
    return float(bad.double().mean()), (float(err.pow(2).mean().sqrt()) / rms if rms > 0 else 0.0)


def rounding_noise(dh, q, k, v, f, i, dtype, chunk_len=0, work_dtype=torch.float64):
    """Per-element noise of the default 16-bit kernels as {name: sigma} (h, dq, dk, dv, df, di); None for fp32.
    ``chunk_len``: the chunk length the kernels ran the sequence in (0: every key tile), which adds the rounding of the
    chunk states."""
    if dtype == torch.float32:
        return None
    sig = O.mlstm_rounding_noise(dh, q, k, v, f, i, dtype, work_dtype=work_dtype, chunk_len=chunk_len)
    return dict(zip(["h"] + GRAD_NAMES, sig))


def combined(a, b):
    """Noise of the difference of two independent evaluations."""
    return {n: (a[n] ** 2 + b[n] ** 2).sqrt() for n in a}


def assert_close(got, ref, dtype, name, sigma=None):
    """``sigma``: the oracle's rounding-noise prediction for this tensor (default 16-bit kernels only, see above)."""
    got = got.detach().cpu().double()
    ref = ref.detach().cpu().double()
    assert got.shape == ref.shape, (name, got.shape, ref.shape)
    assert torch.isfinite(got).all(), f"{name}: non-finite values"
    if dtype == torch.float32:
        assert sigma is None
        rtol, atol = F32_RTOL, F32_ATOL_FRAC * float(ref.abs().max())
    else:
        rtol, atol = HALF_RTOL, HALF_ATOL
    err = (got - ref).abs()
    ref_rms = float(ref.pow(2).mean().sqrt())
    if sigma is not None:
        sigma = sigma.detach().cpu().double().reshape(ref.shape)
    if ref_rms > 0 and ref.numel() >= 64:
        rms = float(err.pow(2).mean().sqrt())
        limit = REL_RMS[dtype] * ref_rms
        if sigma is not None:
            limit = max(limit, 1.25 * float(sigma.pow(2).mean().sqrt()))
        assert rms <= limit, f"{name}: rms error {rms:.3g} > {limit:.3g} (reference rms {ref_rms:.3g})"
    bound = atol + rtol * ref.abs()
    if sigma is not None:
        bound = bound + NOISE_SIGMAS * sigma
    bad = err > bound
    if bool(bad.any()):
        idx = int(torch.argmax(err - bound))
        raise AssertionError(
            f"{name}: {int(bad.sum())}/{bad.numel()} elements outside rtol={rtol} atol={atol:.3g}"
            f"{' + %g sigma' % NOISE_SIGMAS if sigma is not None else ''}; "
            f"max abs err {float(err.max()):.4g} (ref max {float(ref.abs().max()):.4g}); "
            f"worst at flat index {idx}: got {float(got.reshape(-1)[idx]):.6g} ref {float(ref.reshape(-1)[idx]):.6g} "
            f"bound {float(bound.reshape(-1)[idx]):.4g}")


def assert_matches_oracle(dtype, q, k, v, f, i, dh=None, h=None, m=None, b=None, grads=None, chunk_len=0, precise=False,
                          work_dtype=torch.float64, tag=""):
    """Forward outputs (h, m, b) and / or gradients (dq, dk, dv, df, di) of one run against the dense oracle, each under
    the rule of its arithmetic: m and b are fp32 results for every input type; h and the gradients follow ``dtype``,
    with the rounding-noise term for the default 16-bit kernels and without it in split mode (``precise``)."""
    sig = None
    if dtype != torch.float32 and not precise:
        zeros = dh if dh is not None else torch.zeros_like(q)
        sig = rounding_noise(zeros, q, k, v, f, i, dtype, chunk_len, work_dtype)
    s = (lambda n: sig[n]) if sig is not None else (lambda n: None)
    if h is not None or m is not None or b is not None:
        hr, mr, br = O.mlstm_forward_dense(q, k, v, f, i, dtype=work_dtype)
        if m is not None:
            assert_close(m, mr, torch.float32, tag + "m")
        if b is not None:
            assert_close(b, br, torch.float32, tag + "b")
        if h is not None:
            assert_close(h, hr, dtype, tag + "h", s("h"))
    if grads is not None:
        ref = O.mlstm_backward_dense(dh, q, k, v, f, i, dtype=work_dtype, zero_first_df=True)
        for name, g_, r_ in zip(GRAD_NAMES, grads, ref):
            assert_close(g_, r_, dtype, tag + name, s(name))
