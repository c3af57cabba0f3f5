"""Host-side logic of the drop-in (no GPU): tensor construction, dtype rules, view algebra, Module bookkeeping,
error conventions.  Compute ops are device-only in this build and must refuse host tensors loudly."""
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


def test_compute_on_host_tensors_is_refused_loudly():
    a = rp.values([1.0, 2.0, 3.0, 4.0]).reshape([2, 2])
    with pytest.raises(RuntimeError, match="op_matmul operation failed"):
        a.op_matmul(a)
    for call in (lambda: a.op_add(a), lambda: a.op_relu(), lambda: a.op_softmax(), lambda: a.op_sum_all(),
                 lambda: a.op_linear(a), lambda: a.op_cross_entropy_loss([0, 1])):
        with pytest.raises(RuntimeError, match="operation failed"):
            call()
    assert np.allclose(a.mul_scalar(0.5).to_numpy(), [[0.5, 1.0], [1.5, 2.0]])        # initialiser helper stays on the host
    with pytest.raises(RuntimeError, match="op_matmul operation failed"):               # shape errors come first, device or not
        a.op_matmul(rp.zeros([3, 2]))


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
