"""Single-token projections (`based_decode_linear`): against an fp64 matrix product of the same bf16
inputs, and bit for bit against the stand-alone norm / gate kernels followed by the plain projection."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _rand(shape, dev, seed, scale=1.0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(torch.bfloat16).to(dev)


def _check_product(y, x, w, bias=None):
    """|y - exact| within one bf16 rounding of the exact value plus the fp32 summation error."""
    exact = x.double() @ w.double().T
    if bias is not None:
        exact = exact + bias.double()
    mag = x.double().abs() @ w.double().abs().T
    bound = exact.abs() * 2.0 ** -8 + mag * 2.0 ** -17 + 1e-30
    err = (y.double() - exact).abs()
    assert bool((err <= bound).all()), f"max err/bound {(err / bound).max().item():.3f}"


@pytest.mark.parametrize("M", [1, 2, 4, 5, 8, 9, 17, 32])
@pytest.mark.parametrize("N,K", [(1, 8), (3, 64), (100, 256), (64, 520), (1024, 1024), (1536, 1024), (1024, 2048),
                                 (77, 4096), (5000, 1024)])
def test_plain_projection(dev, M, N, K):
    from based_amd import ops

    print(f"decode_linear plain M={M} N={N} K={K}", flush=True)
    x, w, b = _rand((M, K), dev, 1), _rand((N, K), dev, 2, 0.05), _rand((N,), dev, 3)
    _check_product(ops.decode_linear(x, w), x, w)
    _check_product(ops.decode_linear(x, w, b), x, w, b)


def test_lm_head_shape_and_strided_operands(dev):
    from based_amd import ops

    print("decode_linear lm head + strides", flush=True)
    M, N, K = 4, 50280, 1024
    xbig, wbig = _rand((M, 3, K + 64), dev, 4), _rand((N, K + 8), dev, 5, 0.05)
    x, w = xbig[:, 1, 32:32 + K], wbig[:, 8:]
    assert x.stride(0) == 3 * (K + 64) and w.stride(0) == K + 8
    y = ops.decode_linear(x, w)
    _check_product(y, x, w)
    out = torch.full((M, N + 8), 7.0, dtype=torch.bfloat16, device=dev)
    ops.decode_linear(x, w, out=out[:, :N])
    assert torch.equal(out[:, :N], y) and bool((out[:, N:] == 7).all())


@pytest.mark.parametrize("M,N,K,norm", [(12, 20000, 1024, True), (3, 9000, 2048, False), (9, 40000, 64, True),
                                        (32, 50280, 1024, True)])
def test_more_row_groups_than_wavefronts(dev, M, N, K, norm):
    """Launches whose wavefronts walk several row groups (two register sets taking turns), also
    with more activation rows than one tile holds."""
    from based_amd import ops

    print(f"decode_linear rounds M={M} N={N} K={K} norm={norm}", flush=True)
    x, w, b = _rand((M, K), dev, 50), _rand((N, K), dev, 51, 0.05), _rand((N,), dev, 52)
    if norm:
        nw, res = _rand((K,), dev, 53), _rand((M, K), dev, 54).float()
        normed, _ = ops.add_rms_norm(x, res, nw, 1e-5, residual_in_fp32=True)
        y = ops.decode_linear(x, w, b, prologue=ops.PROLOGUE_ADD_RMS_NORM, residual_in=res, norm_weight=nw, eps=1e-5)
        _check_product(y, normed, w, b)
    else:
        _check_product(ops.decode_linear(x, w, b), x, w, b)


@pytest.mark.parametrize("M,N,K", [(1, 48, 64), (4, 1536, 1024), (8, 4096, 1024), (3, 100, 2048), (4, 64, 4096),
                                   (7, 64, 4096), (12, 256, 256)])
@pytest.mark.parametrize("with_residual", [False, True])
def test_norm_prologue_equals_norm_kernel_then_projection(dev, M, N, K, with_residual):
    from based_amd import ops

    print(f"decode_linear norm M={M} N={N} K={K} residual={with_residual}", flush=True)
    x, w, nw = _rand((M, K), dev, 6), _rand((N, K), dev, 7, 0.05), _rand((K,), dev, 8)
    res = _rand((M, K), dev, 9, 3.0).float() * 1.001 if with_residual else None
    normed, r_ref = ops.add_rms_norm(x, res, nw, 1e-5, residual_in_fp32=True)
    y_ref = ops.decode_linear(normed, w)
    r_out = torch.empty(M, K, dtype=torch.float32, device=dev)
    y = ops.decode_linear(x, w, prologue=ops.PROLOGUE_ADD_RMS_NORM, residual_in=res, residual_out=r_out,
                          norm_weight=nw, eps=1e-5)
    assert torch.equal(y, y_ref)
    assert torch.equal(r_out, r_ref)
    y2 = ops.decode_linear(x, w, prologue=ops.PROLOGUE_ADD_RMS_NORM, residual_in=res, norm_weight=nw, eps=1e-5)
    assert torch.equal(y2, y_ref)


@pytest.mark.parametrize("M,N,K", [(1, 16, 8), (4, 1024, 2048), (8, 1024, 2048), (5, 300, 704), (2, 64, 4096), (20, 64, 512)])
def test_swiglu_prologue_equals_gate_kernel_then_projection(dev, M, N, K):
    from based_amd import ops

    print(f"decode_linear swiglu M={M} N={N} K={K}", flush=True)
    u, w = _rand((M, 2 * K), dev, 10, 2.0), _rand((N, K), dev, 11, 0.05)
    y_ref = ops.decode_linear(ops.swiglu(u), w)
    assert torch.equal(ops.decode_linear(u, w, prologue=ops.PROLOGUE_SWIGLU), y_ref)


@pytest.mark.parametrize("M,F,K", [(1, 8, 8), (4, 2048, 1024), (8, 2048, 1024), (5, 104, 520), (9, 64, 2048), (3, 16, 64)])
@pytest.mark.parametrize("norm", [False, True])
def test_swiglu_epilogue_equals_projection_then_gate_kernel(dev, M, F, K, norm):
    from based_amd import ops

    print(f"decode_linear swiglu epilogue M={M} F={F} K={K} norm={norm}", flush=True)
    x, w, b = _rand((M, K), dev, 20), _rand((2 * F, K), dev, 21, 0.2), _rand((2 * F,), dev, 22)
    kw = {}
    if norm:
        kw = dict(prologue=ops.PROLOGUE_ADD_RMS_NORM, norm_weight=_rand((K,), dev, 23),
                  residual_in=_rand((M, K), dev, 24).float())
    for bias in (None, b):
        y_ref = ops.swiglu(ops.decode_linear(x, w, bias, **kw))
        assert torch.equal(ops.decode_linear(x, w, bias, epilogue=ops.EPILOGUE_SWIGLU, **kw), y_ref)


@pytest.mark.parametrize("M,F,K", [(1, 1, 8), (5, 101, 520), (3, 7, 64)])
def test_swiglu_epilogue_odd_widths(dev, M, F, K):
    """Widths the stand-alone gate kernel does not take: against torch's SiLU on the projection."""
    from based_amd import ops

    print(f"decode_linear swiglu epilogue M={M} F={F} K={K}", flush=True)
    x, w = _rand((M, K), dev, 25), _rand((2 * F, K), dev, 26, 0.2)
    p = ops.decode_linear(x, w).float()
    want = p[:, :F] * torch.nn.functional.silu(p[:, F:])
    got = ops.decode_linear(x, w, epilogue=ops.EPILOGUE_SWIGLU).float()
    assert bool(((got - want).abs() <= 2.0 ** -6 * want.abs() + 1e-6).all())


@pytest.mark.parametrize("M,F,K,k", [(1, 8, 64, 3), (4, 2048, 1024, 3), (8, 2048, 1024, 3), (5, 104, 520, 2), (9, 64, 2048, 4),
                                     (20, 16, 256, 3)])
@pytest.mark.parametrize("state_dtype", [torch.bfloat16, torch.float32])
def test_conv_epilogue_equals_projection_then_conv_step(dev, M, F, K, k, state_dtype):
    from based_amd import ops

    print(f"decode_linear conv epilogue M={M} F={F} K={K} k={k} state={state_dtype}", flush=True)
    w, b = _rand((2 * F, K), dev, 31, 0.2), _rand((2 * F,), dev, 32)
    cw, cb = _rand((F, 1, k), dev, 33), _rand((F,), dev, 34)
    nw = _rand((K,), dev, 35)
    s_ref = _rand((M, F, k), dev, 36).to(state_dtype)
    s_got = s_ref.clone()
    for step in range(3):   # consecutive steps roll the state further
        x = _rand((M, K), dev, 40 + step)
        bias, conv_bias = (b, cb) if step != 1 else (None, None)
        kw = dict(prologue=ops.PROLOGUE_ADD_RMS_NORM, norm_weight=nw) if step == 2 else {}
        y_ref = ops.gated_conv_step(ops.decode_linear(x, w, bias, **kw), s_ref, cw, conv_bias)
        y = ops.decode_linear(x, w, bias, epilogue=ops.EPILOGUE_GATED_CONV_STEP, conv_state=s_got, conv_weight=cw,
                              conv_bias=conv_bias, **kw)
        assert torch.equal(y, y_ref), f"step {step}"
        assert torch.equal(s_got, s_ref), f"state after step {step}"


def test_row_index_gathers_table_rows(dev):
    from based_amd import ops

    print("decode_linear row index", flush=True)
    V, K, N = 1000, 1024, 256
    table, w, nw = _rand((V, K), dev, 12), _rand((N, K), dev, 13, 0.05), _rand((K,), dev, 14)
    ids = torch.tensor([5, 999, 0, 5, 123, 77, 42, 998, 1, 2], dtype=torch.int64, device=dev)
    assert torch.equal(ops.decode_linear(table, w, row_index=ids), ops.decode_linear(table[ids], w))
    r1 = torch.empty(ids.numel(), K, dtype=torch.float32, device=dev)
    r2 = torch.empty_like(r1)
    y1 = ops.decode_linear(table, w, prologue=ops.PROLOGUE_ADD_RMS_NORM, norm_weight=nw, residual_out=r1, row_index=ids)
    y2 = ops.decode_linear(table[ids], w, prologue=ops.PROLOGUE_ADD_RMS_NORM, norm_weight=nw, residual_out=r2)
    assert torch.equal(y1, y2) and torch.equal(r1, r2)
    # a token id outside the table: that row is NaN, the others are untouched, nothing faults
    bad = torch.tensor([5, V, 7, -1], dtype=torch.int64, device=dev)
    for kw in ({}, {"prologue": ops.PROLOGUE_ADD_RMS_NORM, "norm_weight": nw}):
        y = ops.decode_linear(table, w, row_index=bad, **kw)
        good = ops.decode_linear(table[torch.tensor([5, 7], device=dev)], w, **kw)
        assert bool(y[1].isnan().all()) and bool(y[3].isnan().all())
        assert torch.equal(y[0], good[0]) and torch.equal(y[2], good[1])


def test_rejects(dev):
    from based_amd import _lib, ops

    x, w = _rand((4, 64), dev, 15), _rand((8, 64), dev, 16)
    with pytest.raises(ValueError):
        ops.decode_linear(_rand((33, 64), dev, 17), w)
    with pytest.raises(ValueError):
        ops.decode_linear(x.float(), w)
    with pytest.raises(ValueError):
        ops.decode_linear(x, w, norm_weight=_rand((64,), dev, 18))
    lib = _lib.lib()
    r = torch.zeros(4, 64, dtype=torch.float32, device=dev)
    y = torch.empty(4, 8, dtype=torch.bfloat16, device=dev)
    nw = _rand((64,), dev, 19)
    # residual_out aliasing residual_in, K beyond 4096, K not a multiple of 8
    tail = (0, None, 0, None, None, 0, None)   # no epilogue, default stream
    assert lib.based_decode_linear(x.data_ptr(), 64, None, 0, w.data_ptr(), 64, None, y.data_ptr(), 8, 4, 8, 64, 1,
                                   r.data_ptr(), 64, r.data_ptr(), 64, nw.data_ptr(), 1e-5, *tail) == 4
    assert lib.based_decode_linear(x.data_ptr(), 4104, None, 0, w.data_ptr(), 4104, None, y.data_ptr(), 8, 4, 8, 4104,
                                   0, None, 0, None, 0, None, 1e-5, *tail) == 1
    assert lib.based_decode_linear(x.data_ptr(), 64, None, 0, w.data_ptr(), 64, None, y.data_ptr(), 8, 4, 8, 60, 0,
                                   None, 0, None, 0, None, 1e-5, *tail) == 1
    # a paired epilogue on an odd number of weight rows / beyond K = 2048, a convolution epilogue without its state
    assert lib.based_decode_linear(x.data_ptr(), 64, None, 0, w.data_ptr(), 64, None, y.data_ptr(), 8, 4, 7, 64, 0,
                                   None, 0, None, 0, None, 1e-5, 1, None, 0, None, None, 0, None) == 1
    assert lib.based_decode_linear(x.data_ptr(), 4096, None, 0, w.data_ptr(), 4096, None, y.data_ptr(), 8, 4, 8, 4096, 0,
                                   None, 0, None, 0, None, 1e-5, 1, None, 0, None, None, 0, None) == 1
    assert lib.based_decode_linear(x.data_ptr(), 64, None, 0, w.data_ptr(), 64, None, y.data_ptr(), 8, 4, 8, 64, 0,
                                   None, 0, None, 0, None, 1e-5, 2, None, 0, None, None, 3, None) == 4
    assert b"decode_linear" in lib.based_hip_last_error()
    with pytest.raises(ValueError):
        ops.decode_linear(x, w, epilogue=ops.EPILOGUE_GATED_CONV_STEP)
    with pytest.raises(ValueError):
        ops.decode_linear(x, w, conv_weight=_rand((4, 1, 3), dev, 20))


def test_overlapping_outputs_are_refused(dev):
    """An output that shares bytes with an input (not only the identical pointer: a view shifted by
    a row) would race between workgroups; the entry point compares byte ranges and refuses."""
    from based_amd import ops

    torch.manual_seed(11)
    M, K, N = 4, 256, 256
    w = torch.randn(N, K, device=dev, dtype=torch.bfloat16)
    nw = torch.ones(K, device=dev, dtype=torch.bfloat16)
    buf = torch.randn(M + 1, K, device=dev, dtype=torch.float32)
    x = torch.randn(M, K, device=dev, dtype=torch.bfloat16)
    with pytest.raises(ValueError):   # residual_out = residual_in shifted by one row
        ops.decode_linear(x, w, prologue=ops.PROLOGUE_ADD_RMS_NORM, residual_in=buf[:M], residual_out=buf[1:],
                          norm_weight=nw)
    xb = torch.randn(M + 1, K, device=dev, dtype=torch.bfloat16)
    with pytest.raises(ValueError):   # y aliases rows of x
        ops.decode_linear(xb[:M], w, out=xb[1:])
    y = ops.decode_linear(xb[:M], w)  # the same call with a fresh output is fine
    assert torch.isfinite(y.float()).all()
