"""oxq_gemv_f32_dev and the OXQ_ROUTE_F32 host route against the reference's f32-activation gemv (oracle:
oxq_ref_gemv, Q/reference/q4_0.rs:82-102, q8_0.rs:77-92, q4_k.rs:135-178, q6_k.rs:108-166, iq4_xs.rs:130-163).
Bar: |y - y_ref| <= 1e-5 * |y_ref|inf (fp32; only the order of the additions differs)."""
import numpy as np
import pytest

import oracle as O
from oxillama_amd import synth

pytestmark = pytest.mark.gpu

F32_TYPES = [O.Q4_0, O.Q8_0, O.Q4_K, O.Q6_K, O.IQ4_XS]
TOL = 1e-5


def run_dev(hip, t, w, x, n_rows, n_cols, **kw):
    import torch
    dev = torch.device("cuda:0")
    dw, dx = torch.from_numpy(w).to(dev), torch.from_numpy(x).to(dev)
    y = torch.full((n_rows,), 5.0, dtype=torch.float32, device=dev)
    hip.HipKernel(t).gemv_f32_dev(dw, dx, y, n_rows, n_cols, **kw)
    torch.cuda.synchronize()
    return y.cpu().numpy()


def assert_close(y, y_ref, what):
    bar = TOL * float(np.abs(y_ref).max())
    err = float(np.abs(y - y_ref).max())
    assert err <= bar, f"{what}: max |diff| {err:.3e} > {bar:.3e}"


# C1 (4096 x 4096), the C2 shapes (14336 x 4096, 4096 x 14336: waves share a row) on a slab of rows the oracle
# finishes in seconds, and rows that do not fill the launch evenly.
@pytest.mark.parametrize("t", F32_TYPES, ids=lambda t: O.NAMES[t])
@pytest.mark.parametrize("n_rows,n_cols", [(4096, 4096), (1500, 4096), (1024, 14336), (37, 14336), (5, 256), (130, 2048)])
def test_gemv_f32_matches_reference(hip, ref, t, n_rows, n_cols):
    w = synth.weights(t, 700 + n_rows, n_rows, n_cols)
    x = synth.normal_f32(701, n_cols)
    y = run_dev(hip, t, w, x, n_rows, n_cols)
    assert_close(y, ref.gemv(t, w, n_rows, n_cols, x), "gemv_f32")


# every payload bit random (all scale / min / index combinations), and activations with a wide range
@pytest.mark.parametrize("t", F32_TYPES, ids=lambda t: O.NAMES[t])
def test_gemv_f32_random_bits(hip, ref, t):
    n_rows, n_cols = 64, 4096
    w = O.random_blocks(t, 710, n_rows, n_cols)
    rng = np.random.default_rng(711)
    x = (rng.standard_normal(n_cols) * np.exp(rng.uniform(-6, 6, n_cols))).astype(np.float32)
    y = run_dev(hip, t, w, x, n_rows, n_cols)
    assert_close(y, ref.gemv(t, w, n_rows, n_cols, x), "gemv_f32 random bits")


# a row that ends inside a block: the reference skips the columns past n_cols (e.g. q4_k.rs:161,168)
@pytest.mark.parametrize("t,n_cols", [(O.Q4_0, 50), (O.Q8_0, 1000), (O.Q4_K, 200), (O.Q4_K, 4000), (O.Q6_K, 300),
                                      (O.Q6_K, 14000), (O.IQ4_XS, 777)], ids=str)
def test_gemv_f32_ragged_rows(hip, ref, t, n_cols):
    n_rows = 19
    bs = O.BLOCK[t][0]
    w = synth.weights(t, 720, n_rows, (n_cols + bs - 1) // bs * bs)  # whole blocks; the row uses the first n_cols columns
    x = synth.normal_f32(721, n_cols)
    y = run_dev(hip, t, w, x, n_rows, n_cols)
    assert_close(y, ref.gemv(t, w, n_rows, n_cols, x), "gemv_f32 ragged")


# rows longer than the register kernel holds (more than 8 steps of 64 units)
@pytest.mark.parametrize("t", [O.Q8_0, O.Q4_K], ids=lambda t: O.NAMES[t])
def test_gemv_f32_long_rows(hip, ref, t):
    n_rows, n_cols = 9, 40960
    w = synth.weights(t, 730, n_rows, n_cols)
    x = synth.normal_f32(731, n_cols)
    y = run_dev(hip, t, w, x, n_rows, n_cols)
    assert_close(y, ref.gemv(t, w, n_rows, n_cols, x), "gemv_f32 long")


def test_gemv_f32_known_answers(hip):
    # Q/reference/q8_0.rs:175-190: d = 1, qs = [1, 1, 1, 0, ...], x = [1, 2, 3, 0, ...] -> 6.0
    x = np.array([1.0, 2.0, 3.0] + [0.0] * 29, dtype=np.float32)
    blk = np.frombuffer(O.make_q8_0_block(1.0, [1, 1, 1] + [0] * 29), dtype=np.uint8).copy()
    y = run_dev(hip, O.Q8_0, blk, x, 1, 32)
    assert y[0] == 6.0


def test_gemv_f32_bias_and_accumulate(hip, ref):
    import torch
    t, n_rows, n_cols = O.Q4_K, 300, 4096
    w = synth.weights(t, 740, n_rows, n_cols)
    x = synth.normal_f32(741, n_cols)
    bias = synth.normal_f32(742, n_rows)
    y_ref = ref.gemv(t, w, n_rows, n_cols, x)
    dev = torch.device("cuda:0")
    y = run_dev(hip, t, w, x, n_rows, n_cols, d_bias=torch.from_numpy(bias).to(dev))
    assert_close(y, y_ref + bias, "bias")
    y = run_dev(hip, t, w, x, n_rows, n_cols, accumulate=True)  # run_dev starts the output at 5.0
    assert_close(y, y_ref + 5.0, "accumulate")


def test_gemv_f32_unsupported_type(hip):
    import torch
    dev = torch.device("cuda:0")
    w = torch.zeros(O.row_bytes(O.Q5_K, 256), dtype=torch.uint8, device=dev)
    with pytest.raises(hip.QuantError) as e:
        hip.HipKernel(O.Q5_K).gemv_f32_dev(w, torch.zeros(256, device=dev), torch.zeros(1, device=dev), 1, 256)
    assert "UNSUPPORTED_TYPE" in str(e.value) or "unsupported" in str(e.value).lower()


@pytest.fixture
def f32_route(hip):
    hip.select_activation_route(hip.ROUTE_F32)
    yield
    hip.select_activation_route(hip.ROUTE_Q8)


# The host-slice route: QuantKernel::gemv / gemm and QuantLinear::forward (linear.rs:77-98) with the reference's numerics
@pytest.mark.parametrize("t", F32_TYPES, ids=lambda t: O.NAMES[t])
def test_host_route_f32(hip, ref, f32_route, t):
    n_rows, n_cols, m = 40, 1024, 3
    w = synth.weights(t, 750, n_rows, n_cols)
    xs = synth.normal_f32(751, m * n_cols)
    k = hip.HipKernel(t)
    qt = hip.QuantTensor(w, [n_rows, n_cols], t)
    assert hip.activation_route() == hip.ROUTE_F32
    y = np.zeros(n_rows, dtype=np.float32)
    k.gemv(qt, xs[:n_cols], y)
    assert_close(y, ref.gemv(t, w, n_rows, n_cols, xs[:n_cols]), "host gemv")
    ys = np.zeros(m * n_rows, dtype=np.float32)
    k.gemm(qt, xs, ys, m, n_rows, n_cols)
    assert_close(ys, ref.gemm(t, w, xs, m, n_rows, n_cols).reshape(-1), "host gemm")


def test_host_route_f32_other_types_fail_loudly(hip, f32_route):
    w = O.random_blocks(O.Q5_K, 760, 4, 256)
    with pytest.raises(hip.QuantError):
        hip.HipKernel(O.Q5_K).gemv(hip.QuantTensor(w, [4, 256], O.Q5_K), np.ones(256, dtype=np.float32),
                                   np.zeros(4, dtype=np.float32))
