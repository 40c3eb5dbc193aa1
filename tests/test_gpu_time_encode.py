"""GPU parity: cos(w*dt+b) through the C ABI vs the CPU oracle.
Tolerance (stated by the task): |y - y_ref| <= 1e-6 * max(1, |y_ref|) with
y_ref = float32(cos(float64(a))), a = fl32(fl32(w*x) + b)."""
import numpy as np
import pytest

from starrygl_amd.lib import _abi
from util import np_of, to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-6


def _w(dim):
    return (1.0 / 10 ** np.linspace(0, 9, dim, dtype=np.float32)).astype(np.float32)


@pytest.mark.parametrize("dim", [100, 16, 7, 1, 172])
@pytest.mark.parametrize("bias", [False, True])
def test_time_encode_i64(oracle, hot, dim, bias):
    rng = np.random.default_rng(dim)
    dt = np.concatenate([np.zeros(3, np.int64), -rng.integers(0, 2_600_000, 4000), rng.integers(0, 2**40, 2000),
                         np.array([1, -1, 2**31, -(2**40)])]).astype(np.int64)
    w = _w(dim)
    b = (rng.standard_normal(dim).astype(np.float32) if bias else np.zeros(dim, np.float32))
    want = oracle.time_encode(dt, w, b)
    got = np_of(hot.time_encode(to_dev(hot, dt), to_dev(hot, w, "f32"), to_dev(hot, b, "f32")))
    err = np.abs(got.astype(np.float64) - want) / np.maximum(1.0, np.abs(want))
    assert err.max() <= TOL, f"max err {err.max()} at {np.unravel_index(err.argmax(), err.shape)}"
    # closed form in float64 on the separately rounded argument
    a = (w[None, :] * dt.astype(np.float32)[:, None]).astype(np.float32) + b[None, :]
    assert np.array_equal(want, np.cos(a.astype(np.float64)).astype(np.float32))


def test_time_encode_f32_input_and_device_count(oracle, hot):
    rng = np.random.default_rng(1)
    dt = (rng.random(5000) * 1e6).astype(np.float32)
    w, b = _w(100), np.zeros(100, np.float32)
    want = oracle.time_encode(dt, w, b, dt_dtype=_abi.DT_F32)
    n_dev = to_dev(hot, np.array([777], dtype=np.int64))
    out = hot.be.zeros((5000, 100), "f32")
    hot.time_encode(to_dev(hot, dt, "f32"), to_dev(hot, w, "f32"), to_dev(hot, b, "f32"), dt_dtype=_abi.DT_F32,
                    out=out, N_dev=n_dev)
    got = np_of(out)
    assert np.abs(got[:777] - want[:777]).max() <= TOL and not got[777:].any()


@pytest.mark.parametrize("dim,rows,live", [
    (100, 50_000, None),        # 10 rows of 25 chunks per trip, tiles of several trips
    (100, 400_000, None),       # the largest tile
    (4, 1_200_000, None),       # one chunk per row: 256 rows per trip
    (1024, 5_000, None),        # 256 chunks per row: one row per trip
    (1028, 300, None),          # 257 chunks per row: more than a block has threads
    (172, 30_011, None),        # 43 chunks per row: 41 threads of a block idle
    (512, 300_000, 290_001),    # more tiles than the capped grid has blocks, live count on the device
])
def test_time_encode_tiles(oracle, hot, dim, rows, live):
    """every tile shape of the kernels (a thread owns one 4-column chunk and walks the rows of a tile; the tile's
    size follows the call's size) against the oracle, bit for bit where the oracle is correctly rounded too."""
    rng = np.random.default_rng(dim + rows)
    dt = rng.integers(-2**40, 2**40, rows).astype(np.int64)
    dt[:5] = [0, 1, -1, 2**40, -(2**40)]
    w, b = _w(dim), rng.standard_normal(dim).astype(np.float32)
    n = rows if live is None else live
    out = hot.be.zeros((rows, dim), "f32")
    hot.time_encode(to_dev(hot, dt), to_dev(hot, w, "f32"), to_dev(hot, b, "f32"), out=out,
                    N_dev=None if live is None else to_dev(hot, np.array([live], dtype=np.int64)))
    got = np_of(out)
    step = 50_000_000 // dim            # the oracle works in float64: bounded pieces
    worst, same, total = 0.0, 0, 0
    for lo in range(0, n, step):
        hi = min(n, lo + step)
        want = oracle.time_encode(dt[lo:hi], w, b)
        err = np.abs(got[lo:hi].astype(np.float64) - want)
        worst = max(worst, float(err.max()))
        same += int((got[lo:hi] == want).sum())
        total += want.size
    assert worst <= 1.2e-7, worst
    assert same / total > 0.99
    assert not got[n:].any()


def test_time_encode_is_within_one_ulp_everywhere(oracle, hot):
    """denser check of the in-kernel cosine: <= 1 ulp (1.2e-7 absolute, |y| <= 1) against the
    correctly rounded oracle over small, mid-range and huge arguments, including the
    library fallback beyond 2^45."""
    rng = np.random.default_rng(0)
    dt = np.concatenate([rng.integers(-50, 50, 2000), rng.integers(-10**7, 10**7, 20_000),
                         rng.integers(-2**44, 2**44, 20_000), rng.integers(-2**62, 2**62, 2000),
                         np.array([2**45, 2**46, -(2**63) + 1, 2**63 - 1])]).astype(np.int64)
    w, b = _w(100), rng.standard_normal(100).astype(np.float32)
    want = oracle.time_encode(dt, w, b)
    got = np_of(hot.time_encode(to_dev(hot, dt), to_dev(hot, w, "f32"), to_dev(hot, b, "f32")))
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    assert err.max() <= 1.2e-7, err.max()
    assert (got == want).mean() > 0.99


def test_time_encoder_module_backward_with_host_and_float_inputs(hot):
    """The module's gradients equal autograd's over cos(Linear(t)) (starrygl/nn/model/time_encoder.py:29-31):
    for an int64 t kept on the host (the kernel reads a device copy, backward must use that copy) and for a
    floating-point t that asks for its own gradient."""
    import torch
    from starrygl_amd.nn.model.time_encoder import TimeEncoder
    torch.manual_seed(0)
    enc = TimeEncoder(16).cuda()
    t_host = torch.randint(0, 1000, (50,))
    enc(t_host).sum().backward()                     # a host tensor: no device mismatch in backward
    gw = enc.w.weight.grad.clone()
    ref = torch.nn.Linear(1, 16).cuda()
    ref.load_state_dict(enc.w.state_dict())
    torch.cos(ref(t_host.cuda().float().reshape(-1, 1))).sum().backward()
    assert torch.allclose(gw, ref.weight.grad, rtol=1e-4, atol=1e-3)
    t = (torch.rand(40, device="cuda") * 100).requires_grad_()
    t2 = t.detach().clone().requires_grad_()
    g = torch.randn(40, 16, device="cuda")
    (enc(t) * g).sum().backward()
    (torch.cos(ref(t2.reshape(-1, 1))) * g).sum().backward()
    assert t.grad is not None and torch.allclose(t.grad, t2.grad, rtol=1e-4, atol=1e-4)
