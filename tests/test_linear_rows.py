"""Linear layers of a decode step on packed operands (tah_linear_pack_weight / tah_linear_pack_rows / tah_linear_rows).

The packed orders are checked element by element against the layout the header documents; the products against
float64 sums of the same bf16 inputs with the roundings the eager modules make (nn.Linear output in bf16, residual
add in bf16, ``act_fn(gate) * up`` of Qwen3MLP.forward with each step in bf16).  Tolerance: the float32 sums run in a
different order from the float64 ones, so a result may land on the neighbouring bf16 value -- 2^-7 relative, and
most elements have to agree exactly.  The CPU tests run the kernels on the CPU execution shim; the GPU tests call the
library through the extension and through ctypes.
"""
import ctypes

import numpy as np
import pytest
import torch

from tests import emu_util

BF = torch.bfloat16


def _rand(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(BF)


def weight_row_of_slot(n, gate_up, tile, c):
    """Row of the [n, k] (or [2n, k]) weight that sits in column slot c of tile `tile` of the packed order."""
    if not gate_up:
        return 16 * tile + c
    if n % 24 == 0:  # groups of 24 output columns, three tiles: gate 0-15 | gate 16-23, up 16-23 | up 0-15
        g, t = divmod(tile, 3)
        if t == 0:
            return 24 * g + c
        if t == 2:
            return n + 24 * g + c
        return 24 * g + 16 + c if c < 8 else n + 24 * g + 16 + (c - 8)
    g, t = divmod(tile, 2)  # groups of 16 output columns: gate tile, up tile
    return (n if t else 0) + 16 * g + c


def unpack_weight(packed, n, k, gate_up):
    """Inverse of the packed order, written from its description: [tiles][k / 32][64 lanes][8]."""
    total = 2 * n if gate_up else n
    p = packed.view(total // 16, k // 32, 64, 8)
    w = torch.empty(total, k, dtype=packed.dtype)
    for tile in range(total // 16):
        for c in range(16):
            row = weight_row_of_slot(n, gate_up, tile, c)
            # lanes c, c + 16, c + 32, c + 48 hold k = 0-7, 8-15, 16-23, 24-31 of every step
            w[row] = p[tile, :, c::16, :].reshape(k)
    return w


def unpack_rows(packed, k):
    """[k / 32][2][64][8] -> [32, k]"""
    p = packed.view(k // 32, 2, 64, 8)
    x = torch.empty(32, k, dtype=packed.dtype)
    for half in range(2):
        for r in range(16):
            x[16 * half + r] = p[:, half, r::16, :].reshape(k)
    return x


def reference(x, w, *, residual=None, gate_up=False, norm_eps=None, bias=None, relu=False, gelu=False, layer_norm=False):
    """float64 sums with the eager modules' bf16 roundings.  ``layer_norm``: the rows go through a LayerNorm without
    scale and shift first (those sit in w and bias), written as the library routine, not as the kernel's fold."""
    xd, wd = x.double(), w.double()
    r = torch.rsqrt((xd ** 2).mean(-1, keepdim=True) + norm_eps) if norm_eps is not None and not layer_norm else 1.0
    if layer_norm:
        xd = torch.nn.functional.layer_norm(xd, xd.shape[-1:], eps=norm_eps)
    if not gate_up:
        y = (r * (xd @ wd.t())).to(BF)
        if bias is not None:
            y = (y.double() + bias.double()).to(BF)
        if residual is not None:
            y = (y.double() + residual.double()).to(BF)
        if gelu:
            return torch.nn.functional.gelu(y.double()).to(BF)
        return torch.relu(y) if relu else y
    n = w.shape[0] // 2
    g = (r * (xd @ wd[:n].t())).to(BF).double()
    u = (r * (xd @ wd[n:].t())).to(BF).double()
    act = (g / (1.0 + torch.exp(-g))).to(BF).double()
    return (act * u).to(BF)


def _close(got, want, exact_share=0.97):
    got, want = got.float(), want.float()
    assert torch.allclose(got, want, rtol=2.0 ** -7, atol=2.0 ** -9), (got - want).abs().max()
    assert (got == want).float().mean() >= exact_share


def _pack_checks(dev):
    from tah_amd import ops
    for n, k, gu in ((48, 96, False), (32, 64, True), (48, 64, True)):
        w = _rand(((2 if gu else 1) * n, k), 3 + n)
        packed = ops.linear_pack_weight(w.to(dev), gate_up=gu).cpu()
        assert packed.shape == (w.numel(),)
        assert torch.equal(unpack_weight(packed, n, k, gu), w)
    # a weight that is a view with a row stride of its own
    big = _rand((32, 256), 9)
    assert torch.equal(unpack_weight(ops.linear_pack_weight(big.to(dev)[:, 64:192]).cpu(), 32, 128, False), big[:, 64:192])
    for rows in (32, 17, 1, 0):
        x = _rand((rows, 160), 5 + rows)
        xp = ops.linear_pack_rows(x.to(dev)).cpu()
        full = unpack_rows(xp, 160)
        assert torch.equal(full[:rows], x) and not full[rows:].any()


CASES = [
    # rows, n, k, kind
    (32, 48, 96, "plain"),       # 3 steps over 8 waves: most waves have no step
    (7, 32, 1024, "residual"),   # 4 steps per wave, any-K kernel
    (17, 16, 2048, "residual"),  # K known at compile time (8 steps per wave)
    (32, 16, 6144, "plain"),     # 24 steps per wave, three chunks
    (20, 32, 352, "plain"),      # 11 steps: uneven shares
    (32, 96, 2048, "gate_up_norm"),   # 24-column groups
    (9, 32, 2048, "gate_up_norm"),    # 16-column groups
    (32, 24, 320, "gate_up"),         # 24-column groups, any K, no norm
    (5, 16, 96, "gate_up_norm"),      # 16-column groups, any K
    # more than 128 column groups: a workgroup takes all 32 rows (below, and up to 16 rows, it takes 16)
    (20, 2080, 96, "residual"),
    (32, 3120, 64, "gate_up_norm"),
    (9, 48, 2048, "plain_norm"),      # an RMSNorm of the rows folded in (an output head behind the final norm)
    (32, 32, 160, "plain_norm"),
    (11, 32, 2048, "bias_relu_norm"),  # first layer of a small MLP behind a folded norm (the decider)
    (32, 48, 96, "bias_relu"),
    (32, 64, 256, "bias_gelu_ln"),     # a layer behind a LayerNorm, GELU last (the learned decider's blocks)
    (13, 2048, 512, "bias_gelu_ln"),   # sixteen rows per workgroup
    (32, 2080, 96, "bias_ln"),         # all 32 rows per workgroup
    (5, 16, 1280, "bias_gelu"),
]


def _linear_case(dev, rows, n, k, kind, seed=0):
    from tah_amd import ops
    gu = kind.startswith("gate_up")
    x = _rand((rows, k), 11 + seed, 1.5)
    w = _rand(((2 if gu else 1) * n, k), 12 + seed, k ** -0.5)
    res = _rand((rows, n), 13 + seed) if kind == "residual" else None
    eps = 1e-6 if kind.endswith("_norm") else None
    bias = _rand((n,), 14 + seed) if kind.startswith("bias") else None
    relu, gelu, ln = "relu" in kind, "gelu" in kind, kind.endswith("_ln")
    if ln:  # rows with a mean of their own, so that a fold that forgets it fails
        x = (x.float() * 0.7 + 0.9 * torch.arange(rows).view(-1, 1) / max(rows, 1) - 0.4).to(BF)
        eps = 1e-5
    want = reference(x, w, residual=res, gate_up=gu, norm_eps=eps, bias=bias, relu=relu, gelu=gelu, layer_norm=ln)
    extra = dict(bias=bias.to(dev), relu=relu, gelu=gelu) if bias is not None else {}
    if ln:
        extra["ln_colsum"] = w.float().sum(-1).to(dev)
    wp = ops.linear_pack_weight(w.to(dev), gate_up=gu)
    xp = ops.linear_pack_rows(x.to(dev))
    yp = torch.full((32 * n,), 7.0, dtype=BF, device=dev) if n % 32 == 0 else None  # the packed form holds whole steps of 32
    if res is not None:  # in place on the residual, as the engine calls it
        h = res.clone().to(dev)
        got = ops.linear_rows(wp, xp, rows, n, k, residual=h, out=h, out_packed=yp)
        assert got.data_ptr() == h.data_ptr()
    else:
        got = ops.linear_rows(wp, xp, rows, n, k, gate_up=gu, out_packed=yp, norm_eps=eps, **extra)
        if relu:
            assert (got.float() >= 0).all() and (got == 0).any()
    got = got.cpu()
    _close(got, want)
    if yp is not None:
        full = unpack_rows(yp.cpu(), n)
        assert torch.equal(full[:rows], got) and not full[rows:].any()   # the packed copy, zero past the last row
        # packed result only
        yp2 = torch.empty_like(yp)
        h2 = res.clone().to(dev) if res is not None else None
        assert ops.linear_rows(wp, xp, rows, n, k, gate_up=gu, residual=h2, out_packed=yp2, want_out=False, norm_eps=eps, **extra) is None
        assert torch.equal(yp2, yp)
    # twice the same: sums run in a fixed order
    again = ops.linear_rows(wp, xp, rows, n, k, gate_up=gu, residual=res.to(dev) if res is not None else None, norm_eps=eps, **extra)
    assert torch.equal(again.cpu(), got)


def _error_checks(dev):
    from tah_amd import ops
    from tah_amd._capi import TahDuoError
    w = _rand((32, 64), 1).to(dev)
    wp = ops.linear_pack_weight(w)
    xp = ops.linear_pack_rows(_rand((4, 64), 2).to(dev))
    with pytest.raises((TahDuoError, RuntimeError)):
        ops.linear_pack_weight(_rand((24, 64), 1).to(dev))            # n % 16
    with pytest.raises((TahDuoError, RuntimeError)):
        ops.linear_pack_weight(_rand((32, 48), 1).to(dev))            # k % 32
    with pytest.raises((TahDuoError, RuntimeError)):
        ops.linear_pack_rows(_rand((33, 64), 1).to(dev))              # more than 32 rows
    with pytest.raises((TahDuoError, RuntimeError)):
        ops.linear_rows(wp, xp, 33, 32, 64)
    with pytest.raises((TahDuoError, RuntimeError)):
        ops.linear_rows(wp, xp, 4, 32, 32)                            # sizes the operands were not packed for
    with pytest.raises((TahDuoError, RuntimeError)):
        ops.linear_rows(wp, xp, 4, 32, 64, norm_eps=1e-5, ln_colsum=torch.zeros(16, device=dev))   # one sum per output column
    with pytest.raises((TahDuoError, RuntimeError)):
        ops.linear_rows(wp, xp, 4, 16, 64, gate_up=True, norm_eps=1e-5, ln_colsum=torch.zeros(16, device=dev))  # no LayerNorm with the gate
    with pytest.raises((TahDuoError, RuntimeError)):
        ops.linear_rows(wp, xp, 4, 16, 64, gate_up=True, residual=_rand((4, 16), 3).to(dev))  # no residual with the gate
    w48 = ops.linear_pack_weight(_rand((48, 64), 4).to(dev))
    with pytest.raises((TahDuoError, RuntimeError)):
        ops.linear_rows(w48, xp, 4, 48, 64, out_packed=torch.empty(32 * 48, dtype=BF, device=dev))  # 48 is not whole steps of 32
    assert ops.linear_rows(wp, xp, 0, 32, 64).shape == (0, 32)


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_packed_orders_on_cpu_shim():
    with emu_util.emulated():
        _pack_checks("cpu")
        _error_checks("cpu")


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
@pytest.mark.parametrize("rows,n,k,kind", CASES)
def test_linear_rows_on_cpu_shim(rows, n, k, kind):
    with emu_util.emulated():
        _linear_case("cpu", rows, n, k, kind)


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_c_abi_refuses_bad_arguments():
    from tah_amd import _capi
    with emu_util.emulated() as lib:
        a = _capi.LinearRowsArgs()
        assert lib.tah_linear_rows(None, None) < 0
        buf = (ctypes.c_uint16 * (32 * 64))()
        addr = ctypes.addressof(buf)
        a.w_packed, a.x_packed, a.out, a.out_row_stride = addr, addr, addr, 32
        a.rows, a.n, a.k, a.kind = 4, 32, 64, 0
        a.rows = 33
        assert lib.tah_linear_rows(ctypes.byref(a), None) < 0
        a.rows, a.n = 4, 24
        assert lib.tah_linear_rows(ctypes.byref(a), None) < 0
        a.n, a.k = 32, 40
        assert lib.tah_linear_rows(ctypes.byref(a), None) < 0
        a.k, a.kind = 64, 5
        assert lib.tah_linear_rows(ctypes.byref(a), None) < 0
        a.kind, a.out = 0, None
        assert lib.tah_linear_rows(ctypes.byref(a), None) < 0          # nothing to write
        a.out, a.x_packed = addr, addr + 2
        assert lib.tah_linear_rows(ctypes.byref(a), None) < 0          # alignment


# ── GPU ──────────────────────────────────────────────────────────────────────────────────────────────────────
@pytest.mark.gpu
def test_packed_orders_gpu():
    _pack_checks("cuda")
    _error_checks("cuda")


@pytest.mark.gpu
@pytest.mark.parametrize("rows,n,k,kind", CASES + [
    (32, 4096, 2048, "plain"), (32, 2048, 2048, "residual"), (32, 6144, 2048, "gate_up_norm"), (32, 2048, 6144, "residual"),
    (13, 1024, 3072, "residual"), (32, 2560, 2560, "plain"), (32, 1600, 1024, "gate_up_norm"),
    (32, 151936, 2048, "plain_norm"), (32, 16384, 512, "plain"), (20, 32000, 1024, "plain_norm"),   # output heads: 32 columns per workgroup
])
def test_linear_rows_gpu(rows, n, k, kind):
    _linear_case("cuda", rows, n, k, kind, seed=n % 7)


@pytest.mark.gpu
def test_linear_rows_through_the_c_abi_gpu():
    """The same call through ctypes, on the library itself."""
    from tah_amd import _capi, _lib, ops
    lib = _capi.bind(ctypes.CDLL(_lib.LIB_PATH))
    rows, n, k = 32, 64, 2048
    x, w, res = _rand((rows, k), 1), _rand((n, k), 2, k ** -0.5), _rand((rows, n), 3)
    dx, dw, h = x.cuda(), w.cuda(), res.clone().cuda()
    wp = torch.empty(n * k, dtype=BF, device="cuda")
    xp = torch.empty(32 * k, dtype=BF, device="cuda")
    yp = torch.empty(32 * n, dtype=BF, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    assert lib.tah_linear_pack_weight(dw.data_ptr(), k, wp.data_ptr(), n, k, _capi.LINEAR_PLAIN, st) == 0
    assert lib.tah_linear_pack_rows(dx.data_ptr(), k, xp.data_ptr(), rows, k, st) == 0
    a = _capi.LinearRowsArgs()
    a.w_packed, a.x_packed, a.residual, a.out, a.out_packed = wp.data_ptr(), xp.data_ptr(), h.data_ptr(), h.data_ptr(), yp.data_ptr()
    a.residual_row_stride = a.out_row_stride = n
    a.rows, a.n, a.k, a.kind = rows, n, k, _capi.LINEAR_PLAIN
    assert lib.tah_linear_rows(ctypes.byref(a), st) == 0
    torch.cuda.synchronize()
    _close(h.cpu(), reference(x, w, residual=res))
    assert torch.equal(unpack_rows(yp.cpu(), n), h.cpu())
    assert torch.equal(ops.linear_pack_weight(dw), wp) and torch.equal(ops.linear_pack_rows(dx), xp)
