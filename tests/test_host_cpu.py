"""Host-side logic of the drop-in (no GPU): tensor construction, dtype rules, view algebra, Module bookkeeping,
error conventions, and the matmul path on host tensors (op_matmul, op_linear, op_add and their gradients), which the
host layer computes in the reference's summation order.  Every other op is device-only and must refuse host tensors loudly."""
import json
import os

import numpy as np
import pytest

import oracle
import recpulse_cuda as rp
from recpulse.module import Linear, Module


def test_constructors_and_properties():
    z = rp.zeros([2, 3])
    assert z.shape == (2, 3) and z.dtype == "float32" and z.device == "cpu" and z.device_id == -1
    assert z.size == 6 and z.ndim == 2 and not z.requires_grad and not z.has_grad and z.grad is None
    assert np.array_equal(z.to_numpy(), np.zeros((2, 3), np.float32))
    o = rp.ones([4], dtype="float64")
    assert o.dtype == "float64" and np.array_equal(o.to_numpy(), np.ones(4))
    v = rp.values([1.0, 2.0, 3.0, 4.0, 5.0, 6.0])
    assert v.shape == (6,) and v.data() == [1.0, 2.0, 3.0, 4.0, 5.0, 6.0]
    assert rp.values([1.5, 2.5], dtype="float64").dtype == "float64"
    with pytest.raises(ValueError):
        rp.zeros([2], dtype="int8")
    with pytest.raises(ValueError):
        rp.zeros([2], device="tpu")


def test_sixteen_bit_storage_uses_the_reference_rounding():
    x = np.array([257.0, -257.0, 1.0 + 2.0 ** -8, 3.14159, 65504.0, 1e-8], dtype=np.float32)
    for name, code in (("bfloat16", oracle.BF16), ("float16", oracle.F16)):
        t = rp.from_numpy(x).to(dtype=name)
        assert t.dtype == name
        want = oracle.to_f64(oracle.narrow(x, code), code)
        assert np.array_equal(t.to(dtype="float32").to_numpy().astype(np.float64), want), name
    assert rp.from_numpy(x).to(dtype="bfloat16").to_numpy().dtype == np.float32       # numpy has no bfloat16
    assert rp.from_numpy(x.astype(np.float16)).dtype == "float16"
    with pytest.raises(TypeError):
        rp.from_numpy(np.arange(4))


def test_views_share_storage_and_follow_stride_algebra():
    base = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    t = rp.from_numpy(base)
    tr = t.transpose(0, 2)
    assert tr.shape == (4, 3, 2) and tr.strides == (1, 4, 12) and not tr.is_contiguous
    assert np.array_equal(tr.to_numpy(), base.transpose(2, 1, 0))
    pm = t.permute([1, 2, 0])
    assert pm.shape == (3, 4, 2) and np.array_equal(pm.to_numpy(), base.transpose(1, 2, 0))
    with pytest.raises(RuntimeError):
        t.permute([0, 0, 1])
    m = rp.from_numpy(base[0])
    assert m.T.shape == (4, 3) and np.array_equal(m.T.to_numpy(), base[0].T)
    with pytest.raises(RuntimeError):
        t.T
    sl = t.slice(start=[0, 1, 0], stop=[2, 3, 4], step=[1, 1, 2])
    assert sl.shape == (2, 2, 2) and np.array_equal(sl.to_numpy(), base[:, 1:3, ::2])
    with pytest.raises(ValueError):
        t.slice(start=[0, 0])
    r = t.reshape([6, -1])
    assert r.shape == (6, 4) and np.array_equal(r.to_numpy(), base.reshape(6, 4))
    assert np.array_equal(tr.reshape([24]).to_numpy(), base.transpose(2, 1, 0).reshape(24))      # non-contiguous source is copied
    assert t.flatten().shape == (24,) and t.view([4, 6]).shape == (4, 6)
    with pytest.raises(RuntimeError):
        t.reshape([5, 5])
    # element i of a 1-D slice, the way the reference's tests read gradients out
    flat = t.flatten()
    assert flat.slice(start=[7], stop=[8]).sum_all() == 7.0


def test_copy_and_grad_flags():
    a = rp.values([1.0, 2.0, 3.0]).requires_grad_(True)
    assert a.requires_grad and not a.has_grad
    b = a.copy()
    assert np.array_equal(b.to_numpy(), a.to_numpy())
    c = rp.zeros([3])
    c.copy_(a)
    assert c.data() == [1.0, 2.0, 3.0]
    with pytest.raises(RuntimeError):
        rp.zeros([4]).copy_(a)
    same = a.to(inplace=True, dtype="float32")
    assert same is a
    a.to(inplace=True, dtype="float64")
    assert a.dtype == "float64" and a.requires_grad                       # metadata survives an in-place move
    with pytest.raises(RuntimeError):
        rp.values([1.0]).backward()                                        # no requires_grad (reference core/tensor.c:221)


def test_host_tensors_compute_matmul_and_add_and_refuse_the_rest():
    """The matmul path runs on host tensors too (reference functional/functional.c:978-1003): op_matmul, op_linear, op_add
    and their gradients.  Every other op is provided on the device only and fails loudly on the host."""
    a = rp.values([1.0, 2.0, 3.0, 4.0]).reshape([2, 2])
    assert np.array_equal(a.op_matmul(a).to_numpy(), [[7.0, 10.0], [15.0, 22.0]])
    assert np.array_equal(a.op_add(a).to_numpy(), [[2.0, 4.0], [6.0, 8.0]])
    for call in (lambda: a.op_relu(), lambda: a.op_softmax(), lambda: a.op_sum_all(), lambda: a.op_cross_entropy_loss([0, 1])):
        with pytest.raises(RuntimeError, match="operation failed"):
            call()
    assert np.allclose(a.mul_scalar(0.5).to_numpy(), [[0.5, 1.0], [1.5, 2.0]])        # initialiser helper stays on the host
    with pytest.raises(RuntimeError, match="op_matmul operation failed"):               # shape errors come first, device or not
        a.op_matmul(rp.zeros([3, 2]))


GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")))


def _host(arr, dtype="float32", grad=False):
    t = rp.from_numpy(np.ascontiguousarray(arr, dtype=np.float64 if dtype == "float64" else np.float32))
    if dtype not in ("float32", "float64"):
        t = t.to(dtype=dtype)
    return t.requires_grad_(True) if grad else t


def _np(t):
    return t.to(dtype="float64").to_numpy()


@pytest.mark.parametrize("dtype", ["float32", "float64", "float16", "bfloat16"])
def test_host_matmul_known_answers_of_the_reference(dtype):
    """The reference's own known answers for the path, on 'cpu' (tests/unit/test_functional.py:281-302,
    tests/autograd/test_matmul_autograd.py:35-128, 215-287)."""
    for key in ("matmul_2x3_3x2", "matmul_identity"):
        c = _host(GOLD[key]["a"], dtype).op_matmul(_host(GOLD[key]["b"], dtype))
        assert np.array_equal(_np(c), np.array(GOLD[key]["c"], dtype=np.float64)), key
    for key in ("backward_a", "backward_both_2x2", "backward_nonsquare_2x4_4x3") + (("backward_f64_2x2",) if dtype == "float64" else ()):
        a, b = _host(GOLD[key]["a"], dtype, grad=True), _host(GOLD[key]["b"], dtype, grad=True)
        a.op_matmul(b).backward()                          # root seeded with ones of its own shape: the gradient of the sum
        assert np.allclose(_np(a.grad), GOLD[key]["da"], rtol=1e-15, atol=0), key
        assert np.allclose(_np(b.grad), GOLD[key]["db"], rtol=1e-15, atol=0), key


@pytest.mark.parametrize("dtype,code", [("float32", oracle.F32), ("float64", oracle.F64), ("float16", oracle.F16), ("bfloat16", oracle.BF16)])
def test_host_matmul_is_the_reference_loop_bit_for_bit(dtype, code):
    """Blocked over the output, but every element still sums its products in the order l = 0 .. k-1 without fused
    multiply-adds: the bits of the reference's i-j-l loop (the oracle, itself pinned to the reference's compiled kernel)
    on ragged shapes, on a transposed view, with a broadcast bias, and for both gradients."""
    rng = np.random.default_rng(7)
    for m, k, n in [(3, 4, 5), (16, 32, 8), (1, 7, 1), (64, 64, 64), (5, 130, 67), (70, 9, 129)]:
        a64, b64, bias64 = rng.uniform(-1, 1, (m, k)), rng.uniform(-1, 1, (k, n)), rng.uniform(-1, 1, (n,))
        a_st, b_st, bias_st = (oracle.to_storage(x, code) for x in (a64, b64, bias64))
        a, b, bias = (_host(oracle.to_f64(x, code), dtype, grad=True) for x in (a_st, b_st, bias_st))
        y = a.op_matmul(b)
        want = oracle.matmul(a_st, b_st, code)
        assert np.array_equal(_np(y), oracle.to_f64(want, code)), (m, k, n)
        z = y.op_add(bias)
        assert np.array_equal(_np(z), oracle.to_f64(oracle.bias_add(want, bias_st, code), code))
        z.backward()
        ones = oracle.to_storage(np.ones((m, n)), code)
        da, db, dbias = oracle.matmul_backward(a_st, b_st, ones, code) + (oracle.reduce_rows(ones, code),)
        assert np.array_equal(_np(a.grad), oracle.to_f64(da, code)) and np.array_equal(_np(b.grad), oracle.to_f64(db, code))
        assert np.array_equal(_np(bias.grad), oracle.to_f64(dbias, code))
        # the same product from a transposed, non-contiguous view of A (reference tests/stress/stress_gradcheck.py:228-243)
        at = _host(oracle.to_f64(np.ascontiguousarray(a_st.T), code), dtype)
        assert np.array_equal(_np(at.transpose(0, 1).op_matmul(b)), oracle.to_f64(want, code))


def test_config1_linear_forward_on_the_host_matches_the_oracle():
    """BASELINE configuration 1 as the reference runs it on its CPU path: Y = X[128,784] @ W[784,256] + b[256], fp32."""
    from recpulse.module import Linear
    rng = np.random.default_rng(0)
    x = rng.uniform(0, 1, (128, 784)).astype(np.float32)
    w = rng.normal(0, np.sqrt(1.0 / 784), (784, 256)).astype(np.float32)
    b = rng.normal(0, 0.1, (256,)).astype(np.float32)
    fc = Linear(784, 256)
    fc.weight.copy_(rp.from_numpy(w)); fc.bias.copy_(rp.from_numpy(b))
    y = fc(rp.from_numpy(x))
    assert np.array_equal(y.to_numpy(), oracle.linear_forward(x, w, b, oracle.F32))


def test_linear_registers_parameters_like_the_reference():
    rp.manual_seed(0)
    fc = Linear(4, 3)
    assert set(fc.tracked) == {"weight", "bias"}
    assert fc.weight.shape == (4, 3) and fc.bias.shape == (3,)
    assert fc.weight.requires_grad and fc.bias.requires_grad
    assert len(fc.parameters()) == 2 and fc.frozen() == {}
    nb = Linear(4, 3, bias=False)
    assert set(nb.tracked) == {"weight"} and nb.bias is None
    w = Linear(1000, 50).weight.to_numpy()
    assert abs(w.std() - (1.0 / 1000) ** 0.5) < 0.004 and abs(w.mean()) < 0.01
    rp.manual_seed(7); w1 = Linear(8, 8).weight.to_numpy()
    rp.manual_seed(7); w2 = Linear(8, 8).weight.to_numpy()
    assert np.array_equal(w1, w2)


def test_nested_modules_flatten_names_and_propagate_mode():
    class Net(Module):
        def __init__(self):
            super().__init__()
            self.fc1 = Linear(4, 8)
            self.fc2 = Linear(8, 2)

    class Outer(Module):
        def __init__(self):
            super().__init__()
            self.body = Net()

    net = Net()
    assert set(net.tracked) == {"fc1.weight", "fc1.bias", "fc2.weight", "fc2.bias"}
    assert set(net._modules) == {"fc1", "fc2"}
    outer = Outer()
    assert "body.fc1.weight" in outer.tracked and "body.fc2" in outer._modules
    assert outer.eval() is outer and not outer._training and not outer.body.fc1._training
    outer.train()
    assert outer.body.fc2._training
    net.to(dtype="float64")
    assert net.fc1.weight.dtype == "float64" and net.fc1.weight.requires_grad
    other = Net()
    other.load_state({"fc1.weight": net.fc1.weight, "unknown": net.fc1.bias})
    assert np.allclose(other.fc1.weight.to_numpy(), net.fc1.weight.to_numpy())
    assert other.fc1.weight.dtype == "float32" and other.fc1.weight.requires_grad
    with pytest.raises(NotImplementedError):
        Module()(1)
