"""Split mode (MLSTM_PRECISE) of the 16-bit kernels on sequences in chunks: chunk states as two terms, hi + lo, through the
four-wave kernels' state phases.  Held to the statement's literal tolerance (rtol 2e-2, atol 2e-3) on every element, against
the fp64 oracle; and the same four-wave kernels in chunks WITHOUT the split (the test switch), against the oracle under the
rule of the default kernels and against the eight-wave / 16x16 kernels."""
import pytest
import torch

from _mlstm_pkg import submodule
from oracle import mlstm_oracle as O
from tests.helpers import GRAD_NAMES, assert_close, assert_matches_oracle, combined, literal_violations, rounding_noise

pytestmark = pytest.mark.gpu

ffi = submodule("_ffi")
mm = submodule("mlstm_matmul")

DT = {"f16": torch.float16, "bf16": torch.bfloat16}


class chunk_length:
    def __init__(self, length):
        self.length = length

    def __enter__(self):
        ffi.set_chunk_length(self.length)

    def __exit__(self, *exc):
        ffi.set_chunk_length(0)


class generic_kernels:
    def __enter__(self):
        self.before = ffi.force_generic_kernels(True)

    def __exit__(self, *exc):
        ffi.force_generic_kernels(self.before)


def dev(*xs):
    return [x.cuda() for x in xs]


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("S,D,L", [(300, 128, 128), (520, 256, 128), (1000, 128, 256), (640, 256, 512), (1100, 256, 0), (2048, 128, 0)])
def test_split_mode_in_chunks_meets_the_literal_bound(dt, S, D, L):
    dtype = DT[dt]
    q, k, v, f, i, dh = O.make_inputs(1, 2, S, D, dtype, seed=S + D + L + 7, f_mean=2.0)
    args = dev(dh, q, k, v, f, i)
    with chunk_length(L):
        assert int(ffi.lib().mlstm_chunk_length_for(S, D, ffi.dtype_code(dtype, True))) > 0
        h, m, b, saved = mm.mlstm_forward_save_hip(*args[1:], precise=True)
        assert saved is not None
        got = mm.mlstm_backward_saved_hip(*args, h, m, b, saved, precise=True)
        again = mm.mlstm_backward_hip(*args, precise=True)            # recomputes the forward, h - T(h) and the states
        h1, m1, b1 = mm.mlstm_forward_hip(*args[1:], precise=True)    # key-major states only
    assert torch.equal(h, h1) and torch.equal(m, m1) and torch.equal(b, b1)
    assert_matches_oracle(dtype, q, k, v, f, i, dh, h=h, m=m, b=b, grads=got, precise=True)
    for n, a_, w_ in zip(GRAD_NAMES, again, got):
        assert torch.equal(a_, w_), n
    with chunk_length(-1):
        plain = mm.mlstm_backward_hip(*args, precise=True)
    for n, g_, p_ in zip(GRAD_NAMES, got, plain):   # two evaluations at 16 bits: the literal bound again
        assert literal_violations(g_, p_.float())[0] == 0.0, n
    assert ffi.lib().mlstm_kernel_error() == 0


def test_split_mode_in_chunks_strong_gates():
    # Input gates that jump by tens of units: the running maximum moves inside and between chunks, states decay to nothing
    # and reappear.  The forward meets the literal bound.  In the gradients single elements are sums of terms 1e4 times
    # their own size (|dq| up to 5e4 next to elements of 1e-2), which 16 significant bits cannot hold: measured, split mode
    # leaves 1e-5 .. 3e-3 of the elements of dq, dk, df outside the literal bound with or without chunks; the test holds the
    # chunked run to that level and to the unchunked run's rms.
    dtype = torch.bfloat16
    S, D = 900, 128
    q, k, v, f, i, dh = O.make_inputs(1, 2, S, D, torch.float32, seed=78)
    i = i * 8.0
    i[..., 400] += 60.0
    f = f * 3.0
    q, k, v, f, i, dh = (x.to(dtype) for x in (q, k, v, f, i, dh))
    ref = O.mlstm_backward_dense(dh, q, k, v, f, i, zero_first_df=True)
    runs = {}
    for L in (-1, 128):
        with chunk_length(L):
            h, m, b, saved = mm.mlstm_forward_save_hip(*dev(q, k, v, f, i), precise=True)
            runs[L] = mm.mlstm_backward_saved_hip(*dev(dh, q, k, v, f, i), h, m, b, saved, precise=True)
        assert_matches_oracle(dtype, q, k, v, f, i, h=h, m=m, precise=True)
    for n, r_, plain, chunked in zip(GRAD_NAMES, ref, runs[-1], runs[128]):
        (bad0, rms0), (bad1, rms1) = literal_violations(plain, r_), literal_violations(chunked, r_)
        assert bad1 <= 5e-3 and rms1 <= 1.05 * rms0 + 1e-4, (n, bad0, rms0, bad1, rms1)


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("S,D,L", [(520, 256, 128), (1000, 128, 256), (1100, 256, 0)])
def test_four_wave_kernels_in_chunks_without_the_split(dt, S, D, L):
    dtype = DT[dt]
    q, k, v, f, i, dh = O.make_inputs(1, 2, S, D, dtype, seed=S + D + L + 9, f_mean=2.0)
    args = dev(dh, q, k, v, f, i)
    with chunk_length(L):
        Lc = int(ffi.lib().mlstm_chunk_length_for(S, D, ffi.dtype_code(dtype)))
        with generic_kernels():
            h, m, b, saved = mm.mlstm_forward_save_hip(*args[1:])
            got = mm.mlstm_backward_saved_hip(*args, h, m, b, saved)
        h8, m8, b8, saved8 = mm.mlstm_forward_save_hip(*args[1:])
        got8 = mm.mlstm_backward_saved_hip(*args, h8, m8, b8, saved8)
    assert Lc > 0
    assert_matches_oracle(dtype, q, k, v, f, i, dh, h=h, m=m, b=b, grads=got, chunk_len=Lc)
    sig = rounding_noise(dh, q, k, v, f, i, dtype, chunk_len=Lc)
    sig = combined(sig, sig)
    assert_close(h, h8.float(), dtype, "h four-wave vs eight-wave", sig["h"])
    for n, g_, p_ in zip(GRAD_NAMES, got, got8):
        assert_close(g_, p_.float(), dtype, n + " four-wave vs eight-wave", sig[n])


def test_saved_buffer_of_another_setting_is_reported():
    dtype = torch.bfloat16
    S, D = 700, 128
    q, k, v, f, i, dh = O.make_inputs(1, 2, S, D, dtype, seed=3, f_mean=2.0)
    args = dev(dh, q, k, v, f, i)
    L = ffi.lib()
    assert L.mlstm_kernel_error() == 0
    with chunk_length(128):
        h, m, b, saved = mm.mlstm_forward_save_hip(*args[1:])
    with chunk_length(128):
        with generic_kernels():   # same sizes, other kernels: the header does not match
            mm.mlstm_backward_saved_hip(*args, h, m, b, saved)
    assert L.mlstm_kernel_error() == -5
    assert L.mlstm_kernel_error() == 0
    with chunk_length(128):
        mm.mlstm_backward_saved_hip(*args, h, m, b, saved)
    assert L.mlstm_kernel_error() == 0


class column_kernel:
    def __init__(self, variant):
        self.variant = variant

    def __enter__(self):
        ffi.set_column_kernel(self.variant)

    def __exit__(self, *exc):
        ffi.set_column_kernel(0)


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("variant", [1, 2, 3])
@pytest.mark.parametrize("B,NH,S,D,L", [(1, 2, 97, 128, -1), (1, 2, 330, 256, -1), (1, 2, 520, 256, 128), (1, 3, 1000, 128, 256), (2, 8, 1536, 256, 0)])
def test_every_column_kernel_against_the_oracle(dt, variant, B, NH, S, D, L):
    """The three column kernels (dK, dV, dI; with the dF pass behind them) that serve the 16-bit types at D = 128 and 256
    -- col16_kernel, cold_kernel (the default) and the generic col_kernel -- on the same inputs: ragged lengths, with and
    without chunks, a multiple of eight heads (the workgroup order by XCD); each under the rule of the default kernels,
    cold_kernel and col_kernel in split mode at the literal bound as well."""
    dtype = DT[dt]
    q, k, v, f, i, dh = O.make_inputs(B, NH, S, D, dtype, seed=S + D + variant, f_mean=2.0)
    args = dev(dh, q, k, v, f, i)
    heads = [(0, 0), (B - 1, NH - 1)]
    with chunk_length(L):
        Lc = int(ffi.lib().mlstm_chunk_length_for(S, D, ffi.dtype_code(dtype)))
        for precise in ([False] if variant == 1 else [False, True]):
            with column_kernel(variant):
                h, m, b, saved = mm.mlstm_forward_save_hip(*args[1:], precise=precise)
                got = mm.mlstm_backward_saved_hip(*args, h, m, b, saved, precise=precise)
            for (bi, hi) in heads:
                one = [x[bi:bi + 1, hi:hi + 1] for x in (q, k, v, f, i, dh)]
                assert_matches_oracle(dtype, *one, grads=[g_[bi:bi + 1, hi:hi + 1] for g_ in got], chunk_len=Lc, precise=precise,
                                      tag=f"kernel {variant} precise={precise} [{bi},{hi}] ")
    assert ffi.lib().mlstm_kernel_error() == 0
