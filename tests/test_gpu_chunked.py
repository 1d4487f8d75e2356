"""The forward of long 16-bit sequences in chunks (matrix state at the chunk ends + the keys of the row's own chunk)
against the CPU oracle and against the unchunked kernels, through the C ABI."""
import pytest
import torch

from _mlstm_pkg import submodule
from oracle import mlstm_oracle as O
from tests.helpers import assert_close, assert_matches_oracle, combined, rounding_noise

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


def dev(*xs):
    return [x.cuda() for x in xs]


def length_in_use(L, S, D, dtype):
    """The chunk length the kernels use under chunk_length(L) (0 = the default for the shape)."""
    with chunk_length(L):
        return int(ffi.lib().mlstm_chunk_length_for(S, D, ffi.dtype_code(dtype)))


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("S,D,L", [(300, 128, 128), (520, 256, 128), (1000, 128, 256), (640, 256, 512), (1100, 256, 0), (2048, 128, 0)])
def test_chunked_forward_matches_oracle_and_unchunked(dt, S, D, L):
    dtype = DT[dt]
    q, k, v, f, i, _ = O.make_inputs(1, 2, S, D, dtype, seed=S + D + L, f_mean=1.0)
    args = dev(q, k, v, f, i)
    with chunk_length(L):
        h, m, b = mm.mlstm_forward_hip(*args)
    with chunk_length(-1):
        h0, m0, b0 = mm.mlstm_forward_hip(*args)
    assert torch.equal(m, m0)
    Lc = length_in_use(L, S, D, dtype)
    assert Lc > 0
    assert_matches_oracle(dtype, q, k, v, f, i, h=h, m=m, b=b, chunk_len=Lc)           # weights and chunk states rounded
    assert_matches_oracle(dtype, q, k, v, f, i, h=h0, tag="unchunked ")
    # the two paths differ by their independent roundings, not more
    z = torch.zeros_like(q)
    sig = combined(rounding_noise(z, q, k, v, f, i, dtype), rounding_noise(z, q, k, v, f, i, dtype, chunk_len=Lc))
    assert_close(h, h0.float(), dtype, "h chunked vs unchunked", sig["h"])


def test_chunked_forward_strong_gates():
    # input gates that jump by tens of units: the running maximum moves inside and between chunks, states decay to
    # nothing and reappear
    dtype = torch.float16
    S, D = 900, 128
    q, k, v, f, i, _ = O.make_inputs(1, 2, S, D, torch.float32, seed=77)
    i = i * 8.0
    i[..., 400] += 60.0
    f = f * 3.0
    q, k, v, f, i = (x.to(dtype) for x in (q, k, v, f, i))
    with chunk_length(128):
        h, m, b = mm.mlstm_forward_hip(*dev(q, k, v, f, i))
    assert_matches_oracle(dtype, q, k, v, f, i, h=h, m=m, chunk_len=128)


@pytest.mark.parametrize("dt", ["f16", "bf16"])
def test_chunked_gated_forward_and_backward_recompute(dt):
    dtype = DT[dt]
    S, D = 700, 128
    q, k, v, f, i, dh, o = O.make_inputs(1, 2, S, D, dtype, seed=31, f_mean=2.0, with_o=True)
    with chunk_length(256):
        hg, h, m, b = mm.mlstm_forward_gated_hip(*dev(q, k, v, f, i, o))
        got = mm.mlstm_backward_hip(*dev(dh, q, k, v, f, i))        # recomputes h, m, b with the chunked forward
    with chunk_length(-1):
        ref = mm.mlstm_backward_hip(*dev(dh, q, k, v, f, i))
    sig = rounding_noise(torch.zeros_like(q), q, k, v, f, i, dtype, chunk_len=256)
    assert_close(hg, O.mlstm_scan_dense(q, k, v, f, i, o), dtype, "h_gated", sig["h"] * torch.nn.functional.silu(o.double()).abs())
    for name, a, r in zip(["dq", "dk", "dv", "df", "di"], got, ref):
        d = (a.float() - r.float()).pow(2).mean().sqrt() / r.float().pow(2).mean().sqrt()
        assert float(d) < (8e-3 if dtype == torch.bfloat16 else 1.5e-3), (name, float(d))


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("S,D,L", [(300, 128, 128), (520, 256, 128), (1000, 128, 256), (1100, 256, 0)])
@pytest.mark.parametrize("with_fwd", [True, False])
def test_chunked_backward_matches_oracle(dt, S, D, L, with_fwd):
    # the dQ pass takes what lies before a row's chunk from the (value-major) state; dK, dV, dF, dI walk all the queries
    dtype = DT[dt]
    q, k, v, f, i, dh = O.make_inputs(1, 2, S, D, dtype, seed=S + D + L + 1, f_mean=2.0)
    args = dev(dh, q, k, v, f, i)
    with chunk_length(L):
        fwd = mm.mlstm_forward_hip(*args[1:]) if with_fwd else ()
        got = mm.mlstm_backward_hip(*args, *fwd)
    with chunk_length(-1):
        plain = mm.mlstm_backward_hip(*args)
    Lc = length_in_use(L, S, D, dtype)
    assert_matches_oracle(dtype, q, k, v, f, i, dh, grads=got, chunk_len=Lc)
    sig = combined(rounding_noise(dh, q, k, v, f, i, dtype), rounding_noise(dh, q, k, v, f, i, dtype, chunk_len=Lc))
    for name, g, p in zip(["dq", "dk", "dv", "df", "di"], got, plain):
        assert_close(g, p.float(), dtype, name + " chunked vs unchunked", sig[name])


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("S,D,L", [(520, 256, 128), (1000, 128, 256), (200, 128, 0)])
def test_saved_states_give_the_same_backward(dt, S, D, L):
    dtype = DT[dt]
    q, k, v, f, i, dh = O.make_inputs(1, 2, S, D, dtype, seed=S + D + L + 2, f_mean=2.0)
    args = dev(dh, q, k, v, f, i)
    with chunk_length(L):
        h, m, b, saved = mm.mlstm_forward_save_hip(*args[1:])
        h0, m0, b0 = mm.mlstm_forward_hip(*args[1:])
        assert (saved is None) == (S < 1024 and L == 0)
        assert torch.equal(h, h0) and torch.equal(m, m0) and torch.equal(b, b0)
        got = mm.mlstm_backward_saved_hip(*args, h, m, b, saved)
        want = mm.mlstm_backward_hip(*args, h, m, b)      # forms the states again
        for name, a, w in zip(["dq", "dk", "dv", "df", "di"], got, want):
            assert torch.equal(a, w), name
        # through autograd
        ins = [x.clone().requires_grad_(True) for x in args[1:]]
        mm.Triton_mLSTM.apply(*ins).backward(args[0])
        for name, x, w in zip(["dq", "dk", "dv", "df", "di"], ins, want):
            assert torch.equal(x.grad, w), name
        if saved is not None:   # a saved buffer that is too small is refused
            with pytest.raises(ValueError):
                mm.mlstm_backward_saved_hip(*args, h, m, b, saved[:-256])


@pytest.mark.parametrize("B,NH,S,D", [(2, 4, 1536, 256), (2, 8, 2560, 128), (1, 8, 1024, 256), (3, 8, 2048, 128)])
def test_workgroup_order_over_many_heads_changes_nothing(B, NH, S, D):
    # With a multiple of 8 heads the tile kernels deal their workgroups out by XCD, in sets of (head, chunk) groups that
    # may leave a smaller last set; a head on its own takes the plain order.  No kernel adds across workgroups in an
    # order that depends on the launch order, so the results are the same bits.
    dtype = torch.bfloat16
    g = torch.Generator(device="cuda").manual_seed(B * 1000 + S + D)
    mk = lambda *s: torch.randn(s, generator=g, device="cuda")
    q, k, v, dh = (mk(B, NH, S, D).to(dtype) for _ in range(4))
    f, i = (mk(B, NH, S) + 3.0).to(dtype), mk(B, NH, S).to(dtype)
    h, m, b, saved = mm.mlstm_forward_save_hip(q, k, v, f, i)
    assert saved is not None
    grads = mm.mlstm_backward_saved_hip(dh, q, k, v, f, i, h, m, b, saved)
    for bi, hi in [(0, 0), (B - 1, NH - 1), (B // 2, NH // 2 + 1)]:
        one = [x[bi:bi + 1, hi:hi + 1].contiguous() for x in (dh, q, k, v, f, i)]
        h1, m1, b1, s1 = mm.mlstm_forward_save_hip(*one[1:])
        assert torch.equal(h1[0, 0], h[bi, hi]) and torch.equal(m1[0, 0], m[bi, hi]) and torch.equal(b1[0, 0], b[bi, hi])
        g1 = mm.mlstm_backward_saved_hip(*one, h1, m1, b1, s1)
        for name, a, w in zip(["dq", "dk", "dv", "df", "di"], g1, grads):
            assert torch.equal(a[0, 0], w[bi, hi]), (name, bi, hi)


def test_chunk_length_is_validated_and_sizes_follow():
    L = ffi.lib()
    assert L.mlstm_set_chunk_length(100) == -1
    try:
        ffi.set_chunk_length(-1)
        off = L.mlstm_workspace_bytes(ffi.OP_FORWARD, 1, 2, 4096, 256, ffi.BF16)
        ffi.set_chunk_length(512)
        on = L.mlstm_workspace_bytes(ffi.OP_FORWARD, 1, 2, 4096, 256, ffi.BF16)
        assert on >= off + 2 * 7 * 256 * 256 * 6
        assert L.mlstm_workspace_bytes(ffi.OP_FORWARD, 1, 2, 4096, 64, ffi.BF16) == L.mlstm_workspace_bytes(ffi.OP_FORWARD, 1, 2, 4096, 64, ffi.F16)
    finally:
        ffi.set_chunk_length(0)


def test_chunked_forward_at_the_headline_shape():
    """B4 H8 S4096 D256 bf16 (448 state workgroups, two rounds on the chip) is beyond the CPU oracle: the chunked forward
    must be finite, repeatable bit for bit, and agree with the unchunked kernels up to the rounding of the states."""
    dtype = torch.bfloat16
    g = torch.Generator(device="cuda").manual_seed(5)
    B, NH, S, D = 4, 8, 4096, 256
    mk = lambda *s: torch.randn(s, generator=g, device="cuda", dtype=torch.float32)
    q, k, v = (mk(B, NH, S, D).to(dtype) for _ in range(3))
    f, i = (mk(B, NH, S) + 3.0).to(dtype), mk(B, NH, S).to(dtype)
    with chunk_length(-1):
        h0, m0, b0 = mm.mlstm_forward_hip(q, k, v, f, i)
    for L in (0, 256, 1024):
        with chunk_length(L):
            h, m, b = mm.mlstm_forward_hip(q, k, v, f, i)
            h2, _, b2 = mm.mlstm_forward_hip(q, k, v, f, i)
        assert bool(torch.isfinite(h).all()) and torch.equal(h, h2) and torch.equal(b, b2)
        assert torch.equal(m, m0)
        d = h.float() - h0.float()
        assert float(d.pow(2).mean().sqrt() / h0.float().pow(2).mean().sqrt()) < 2e-3, L
        assert float((b - b0).pow(2).mean().sqrt() / b0.pow(2).mean().sqrt()) < 1e-5, L


SMALL = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


@pytest.mark.parametrize("dt,S,D,L", [("f32", 1100, 64, 128), ("f32", 2048, 64, 0), ("f32", 900, 128, 256), ("f32", 1300, 128, 0),
                                      ("bf16", 1100, 64, 128), ("f16", 2048, 64, 0), ("bf16", 1500, 64, 0), ("f16", 700, 64, 256)])
def test_small_shapes_in_chunks(dt, S, D, L):
    # fp32 (D = 64, 128) and the 16-bit types at D = 64: chunk sums by plain multiply-adds, one carry for both state
    # layouts, the four-wave tile kernels in chunk mode.  fp32 is held to its own bound (every element, rtol 1e-4).
    dtype = SMALL[dt]
    q, k, v, f, i, dh = O.make_inputs(1, 2, S, D, dtype, seed=S + D + L + 5, f_mean=2.0)
    args = dev(dh, q, k, v, f, i)
    Lc = length_in_use(L, S, D, dtype)
    assert Lc > 0 and (L == 0 or Lc == L)
    with chunk_length(L):
        h, m, b, saved = mm.mlstm_forward_save_hip(*args[1:])
        assert saved is not None
        got = mm.mlstm_backward_saved_hip(*args, h, m, b, saved)
        again = mm.mlstm_backward_hip(*args, h, m, b)            # forms the states again
        h2, m2, b2 = mm.mlstm_forward_hip(*args[1:])
    assert torch.equal(h, h2) and torch.equal(m, m2) and torch.equal(b, b2)
    for name, a, w in zip(["dq", "dk", "dv", "df", "di"], got, again):
        assert torch.equal(a, w), name
    assert_matches_oracle(dtype, q, k, v, f, i, dh, h=h, m=m, b=b, grads=got, chunk_len=Lc)
    with chunk_length(-1):
        h0, m0, b0 = mm.mlstm_forward_hip(*args[1:])
        plain = mm.mlstm_backward_hip(*args, h0, m0, b0)
    assert torch.equal(m, m0)
    sig = combined(rounding_noise(dh, q, k, v, f, i, dtype), rounding_noise(dh, q, k, v, f, i, dtype, chunk_len=Lc)) if dtype != torch.float32 else None
    for name, g, p in zip(["h", "dq", "dk", "dv", "df", "di"], [h, *got], [h0, *plain]):
        assert_close(g, p.float(), dtype, name + " chunked vs unchunked", sig[name] if sig else None)


@pytest.mark.parametrize("dt", ["f16", "bf16"])
def test_split_mode_in_chunks_at_head_dimension_64(dt):
    # split mode at D = 64: two-term states from the element-wise carry, the literal bound
    dtype = SMALL[dt]
    S, D = 1100, 64
    q, k, v, f, i, dh = O.make_inputs(1, 2, S, D, dtype, seed=411, f_mean=2.0)
    args = dev(dh, q, k, v, f, i)
    with chunk_length(256):
        h, m, b, saved = mm.mlstm_forward_save_hip(*args[1:], precise=True)
        got = mm.mlstm_backward_saved_hip(*args, h, m, b, saved, precise=True)
    assert_matches_oracle(dtype, q, k, v, f, i, dh, h=h, m=m, b=b, grads=got, chunk_len=256, precise=True)


def test_fp32_default_chunk_length_and_many_heads():
    # the default for fp32 is the shortest chunk; a batch of heads gives the bits of its heads run alone
    assert length_in_use(0, 2048, 64, torch.float32) == 128 and length_in_use(0, 1023, 64, torch.float32) == 0
    assert length_in_use(0, 4096, 64, torch.bfloat16) == 256 and length_in_use(0, 4096, 128, torch.bfloat16) == 512
    g = torch.Generator(device="cuda").manual_seed(5)
    B, NH, S, D = 2, 3, 1536, 64
    q, k, v, dh = (torch.randn(B, NH, S, D, generator=g, device="cuda") for _ in range(4))
    f, i = torch.randn(B, NH, S, generator=g, device="cuda") + 3.0, torch.randn(B, NH, S, generator=g, device="cuda")
    h, m, b, saved = mm.mlstm_forward_save_hip(q, k, v, f, i)
    grads = mm.mlstm_backward_saved_hip(dh, q, k, v, f, i, h, m, b, saved)
    one = [x[1:2, 2:3].contiguous() for x in (dh, q, k, v, f, i)]
    h1, m1, b1, s1 = mm.mlstm_forward_save_hip(*one[1:])
    g1 = mm.mlstm_backward_saved_hip(*one, h1, m1, b1, s1)
    assert torch.equal(h1[0, 0], h[1, 2]) and torch.equal(b1[0, 0], b[1, 2])
    for name, a, w in zip(["dq", "dk", "dv", "df", "di"], g1, grads):
        assert torch.equal(a[0, 0], w[1, 2]), name


class state_kernel:
    def __init__(self, variant):
        self.variant = variant

    def __enter__(self):
        ffi.set_state_kernel(self.variant)

    def __exit__(self, *exc):
        ffi.set_state_kernel(0)


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("B,NH,S,D,L", [(1, 2, 1100, 256, 256), (1, 3, 1573, 128, 512), (2, 8, 2048, 256, 0), (1, 2, 1000, 128, 128), (1, 1, 4096 + 70, 128, 0)])
def test_one_pass_state_kernel(dt, B, NH, S, D, L):
    # the chunk states by the kernel that walks a head's chunks in order ((D / 64) * 2 workgroups per head, hand-counted
    # direct loads): forward and backward against the oracle, and against the two-kernel form within the rounding of the
    # weighted operand (the two weight different operands); ragged last chunks, head counts with and without the XCD order
    dtype = DT[dt]
    q, k, v, f, i, dh = O.make_inputs(B, NH, S, D, dtype, seed=S + D + L + 9, f_mean=2.0)
    args = dev(dh, q, k, v, f, i)
    Lc = length_in_use(L, S, D, dtype)
    outs = []
    for variant in (2, 1):
        with chunk_length(L), state_kernel(variant):
            h, m, b, saved = mm.mlstm_forward_save_hip(*args[1:])
            got = mm.mlstm_backward_saved_hip(*args, h, m, b, saved)
            again = mm.mlstm_backward_hip(*args, h, m, b)
        assert ffi.lib().mlstm_kernel_error() == 0
        for name, a, w in zip(["dq", "dk", "dv", "df", "di"], got, again):
            assert torch.equal(a, w), name
        outs.append([h, m, b, *got])
    sl = lambda x: x[B - 1:B, NH - 1:NH]
    h, m, b, *got = outs[0]
    assert_matches_oracle(dtype, *(sl(x) for x in (q, k, v, f, i, dh)), h=sl(h), m=sl(m), b=sl(b), grads=[sl(g) for g in got], chunk_len=Lc)
    one = rounding_noise(sl(dh), *(sl(x) for x in (q, k, v, f, i)), dtype, chunk_len=Lc)
    sig = combined(one, one)
    for name, x, y in zip(["h", "m", "b", "dq", "dk", "dv", "df", "di"], outs[0], outs[1]):
        if name in ("m", "b"):
            assert_close(sl(x), sl(y).double(), torch.float32, name + " one pass vs two kernels")
        else:
            assert_close(sl(x), sl(y).float(), dtype, name + " one pass vs two kernels", sig[name])
