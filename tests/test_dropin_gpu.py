"""The drop-in Python surface (`recpulse_cuda`, `recpulse.module`) on the GPU.

The cases follow the reference's own tests for the matmul path (each test names
the one it mirrors), run with device='cuda' so that every op goes host C++ ->
C ABI -> HIP kernel, and are checked against the known answers, finite
differences, torch autograd in float64 and the CPU oracle.
"""
import json
import os

import numpy as np
import pytest

import oracle
import recpulse_cuda as rp
from recpulse.module import Linear, Module

pytestmark = pytest.mark.gpu
GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")))
DTYPES = ["float32", "float64", "float16", "bfloat16"]


def dev(arr, dtype="float64", grad=False):
    """numpy -> device tensor of `dtype` (bfloat16 travels through float32, as in the reference's tests)."""
    t = rp.from_numpy(np.ascontiguousarray(arr, dtype=np.float64 if dtype == "float64" else np.float32)).to(device="cuda", dtype=dtype)
    return t.requires_grad_(True) if grad else t


def host(t):
    return t.to(device="cpu", dtype="float64").to_numpy()


# ---- reference tests/unit/test_functional.py:281-302, tests/unit/test_half_precision_full.py:267-274
@pytest.mark.parametrize("dtype", DTYPES)
def test_matmul_forward_known_answers(dtype):
    g = GOLD["matmul_2x3_3x2"]
    a = rp.values([1, 2, 3, 4, 5, 6], dtype=dtype, device="cuda").reshape([2, 3])
    b = rp.values([1, 2, 3, 4, 5, 6], dtype=dtype, device="cuda").reshape([3, 2])
    c = a.op_matmul(b)
    assert c.shape == (2, 2) and c.dtype == dtype and c.device == "cuda:0"
    assert np.array_equal(host(c), np.array(g["c"], dtype=np.float64))
    assert host(c).sum() == g["c_sum"]
    i2 = rp.values([1, 0, 0, 1], dtype=dtype, device="cuda").reshape([2, 2])
    b2 = rp.values([5, 6, 7, 8], dtype=dtype, device="cuda").reshape([2, 2])
    assert np.array_equal(host(i2.op_matmul(b2)), np.array(GOLD["matmul_identity"]["c"], dtype=np.float64))


# ---- reference tests/autograd/test_matmul_autograd.py:35-128, 215-287
@pytest.mark.parametrize("dtype", DTYPES)
def test_matmul_backward_known_answers(dtype):
    for key in ("backward_a", "backward_both_2x2", "backward_nonsquare_2x4_4x3"):
        g = GOLD[key]
        a = dev(g["a"], dtype, grad=True); b = dev(g["b"], dtype, grad=True)
        s = a.op_matmul(b).op_sum_all()
        s.backward()
        assert a.grad.shape == tuple(np.shape(g["a"])) and a.grad.dtype == dtype
        assert np.array_equal(host(a.grad), np.array(g["da"], dtype=np.float64)), key
        assert np.array_equal(host(b.grad), np.array(g["db"], dtype=np.float64)), key
    g = GOLD["backward_f64_2x2"]
    a = dev(g["a"], "float64", grad=True); b = dev(g["b"], "float64", grad=True)
    s = a.op_matmul(b).op_sum_all()
    assert abs(s.sum_all() - g["c_sum"]) < 1e-10
    s.backward()
    assert np.max(np.abs(host(a.grad) - np.array(g["da"]))) < 1e-10
    assert np.max(np.abs(host(b.grad) - np.array(g["db"]))) < 1e-10
    only_b = dev(GOLD["backward_a"]["a"], "float64")
    bb = dev(GOLD["backward_a"]["b"], "float64", grad=True)
    only_b.op_matmul(bb).op_sum_all().backward()
    assert not only_b.has_grad and bb.has_grad


def _numeric_grad(fn, arrays, idx, eps=1e-5):
    base = [a.copy() for a in arrays]
    g = np.zeros_like(base[idx])
    it = np.nditer(base[idx], flags=["multi_index"])
    for _ in it:
        i = it.multi_index
        plus = [a.copy() for a in base]; plus[idx][i] += eps
        minus = [a.copy() for a in base]; minus[idx][i] -= eps
        g[i] = (fn(plus) - fn(minus)) / (2 * eps)
    return g


# ---- reference tests/stress/stress_gradcheck.py:214-243 (central differences eps 1e-5, tol 1e-4; CPU/GPU parity there, float64 here)
def test_gradcheck_plain_and_transposed_noncontiguous():
    rng = np.random.default_rng(50)
    w = rng.uniform(0.5, 1.5, (3, 2))

    def run(arrays, transposed):
        a = dev(arrays[0], "float64", grad=True); b = dev(arrays[1], "float64", grad=True)
        left = a.transpose(0, 1) if transposed else a
        assert left.is_contiguous != transposed
        y = left.op_matmul(b)
        # weighted sum(y * w) from the ops this build has: for each column j, w[:, j]ᵀ · (y · e_j)
        total = None
        for j in range(2):
            col = y.op_matmul(dev(np.eye(2)[:, j:j + 1] * 1.0, "float64"))            # [3,1] column j
            wcol = dev(w[:, j:j + 1].T, "float64")                                     # [1,3]
            term = wcol.op_matmul(col)                                                 # [1,1]
            total = term if total is None else total.op_add(term)
        total.op_sum_all().backward()
        return host(a.grad), host(b.grad), float(host(total).sum())

    for transposed, ashape in ((False, (3, 4)), (True, (4, 3))):
        a = rng.uniform(-1, 1, ashape); b = rng.uniform(-1, 1, (4, 2))
        ga, gb, val = run([a, b], transposed)
        f = lambda arrs: float((((arrs[0].T if transposed else arrs[0]) @ arrs[1]) * w).sum())
        assert abs(val - f([a, b])) < 1e-10
        assert np.max(np.abs(ga - _numeric_grad(f, [a, b], 0))) < 1e-4
        assert np.max(np.abs(gb - _numeric_grad(f, [a, b], 1))) < 1e-4


# ---- reference tests/autograd/test_matmul_autograd.py:186-213
def test_matmul_mul_scalar_sum_chain():
    a = dev([[1, 2], [3, 4]], "float64", grad=True); b = dev([[1, 0], [0, 1]], "float64")
    a.op_matmul(b).op_mul_scalar(2.0).op_sum_all().backward()
    assert np.max(np.abs(host(a.grad) - 2.0 * np.ones((2, 2)) @ np.eye(2))) < 1e-10


def test_gradient_accumulates_until_zero_grad():
    a = dev([[1, 2], [3, 4]], "float32", grad=True); b = dev([[5, 6], [7, 8]], "float32", grad=True)
    a.op_matmul(b).op_sum_all().backward()
    first = host(a.grad)
    a.op_matmul(b).op_sum_all().backward()                 # second graph: the GEMM accumulates into the existing grad
    assert np.array_equal(host(a.grad), 2 * first) and np.array_equal(host(b.grad), 2 * np.array([[4, 4], [6, 6]]))
    a.zero_grad()
    assert not a.has_grad and a.grad is None               # freed, not zero-filled (reference tests/integration/test_module.py:154-164)
    g = a.grad
    a.op_matmul(b).op_sum_all().backward()
    assert np.array_equal(host(a.grad), first) and g is None
    twice = a.op_matmul(b)
    y = twice.op_add(twice)                                 # one tensor used twice: both contributions reach it
    a.zero_grad(); b.zero_grad()
    y.op_sum_all().backward()
    assert np.array_equal(host(a.grad), 2 * first)


# ---- reference tests/autograd/test_complex_chains.py:43-120, tests/integration/test_module.py:45-62
def test_linear_forward_and_finite_differences():
    rng = np.random.default_rng(51)
    rp.manual_seed(3)
    fc = Linear(5, 3).to(device="cuda", dtype="float64")
    assert fc.weight.device == "cuda:0" and fc.weight.requires_grad and fc.bias.requires_grad
    x = rng.uniform(-1, 1, (4, 5)); w = host(fc.weight); b = rng.normal(0, 1, 3)
    fc.load_state({"bias": dev(b, "float64")})
    xt = dev(x, "float64", grad=True)
    y = fc(xt)
    assert y.shape == (4, 3) and np.max(np.abs(host(y) - (x @ w + b))) < 1e-12
    assert np.array_equal(host(fc.forward_two_ops(xt)), host(y))        # fused epilogue == matmul then broadcasting add
    y.op_sum_all().backward()
    f = lambda arrs: float((arrs[0] @ arrs[1] + arrs[2]).sum())
    assert np.max(np.abs(host(xt.grad) - _numeric_grad(f, [x, w, b], 0))) < 1e-4
    assert np.max(np.abs(host(fc.weight.grad) - _numeric_grad(f, [x, w, b], 1))) < 1e-4
    assert np.max(np.abs(host(fc.bias.grad) - _numeric_grad(f, [x, w, b], 2))) < 1e-4
    assert fc.bias.grad.shape == (3,)
    fc.zero_grad()
    assert not fc.weight.has_grad and not fc.bias.has_grad
    nb = Linear(5, 3, bias=False).to(device="cuda")
    assert nb(dev(x, "float32")).shape == (4, 3)


# ---- reference tests/stress/stress_gradcheck.py:549-566, tests/stress/stress_torch_parity.py:150-171 (rtol 1e-7 in float64)
def test_two_layer_composite_matches_torch():
    import torch
    rng = np.random.default_rng(52)
    x, w1, w2 = rng.uniform(-1, 1, (6, 5)), rng.uniform(-1, 1, (5, 7)), rng.uniform(-1, 1, (7, 3))
    xt, w1t, w2t = (dev(a, "float64", grad=True) for a in (x, w1, w2))
    out = xt.op_matmul(w1t).op_relu().op_matmul(w2t).op_mean_all()
    out.backward()
    tx, t1, t2 = (torch.tensor(a, requires_grad=True) for a in (x, w1, w2))
    (torch.relu(tx @ t1) @ t2).mean().backward()
    for got, want in ((xt, tx), (w1t, t1), (w2t, t2)):
        np.testing.assert_allclose(host(got.grad), want.grad.numpy(), rtol=1e-7, atol=1e-12)


class MLP(Module):
    def __init__(self, dims):
        super().__init__()
        self.n = len(dims) - 1
        for i in range(self.n):
            setattr(self, f"fc{i + 1}", Linear(dims[i], dims[i + 1]))

    def forward(self, x):
        for i in range(self.n):
            x = getattr(self, f"fc{i + 1}")(x)
            if i + 1 < self.n:
                x = x.op_relu()
        return x


# ---- benchmark configuration 2 through the Python API: every dW, db and dX against the CPU oracle (reference autograd order)
def test_config2_mlp_through_modules_matches_oracle():
    rng = np.random.default_rng(1)
    dims = [784, 256, 128, 10]; batch = 256
    x = rng.uniform(0, 1, (batch, dims[0])).astype(np.float32)
    ws = [rng.normal(0, np.sqrt(2.0 / dims[i]), (dims[i], dims[i + 1])).astype(np.float32) for i in range(3)]
    bs = [np.zeros(dims[i + 1], np.float32) for i in range(3)]
    y = rng.integers(0, 10, batch)
    net = MLP(dims).to(device="cuda")
    net.load_state({f"fc{i + 1}.weight": rp.from_numpy(ws[i]) for i in range(3)})
    net.load_state({f"fc{i + 1}.bias": rp.from_numpy(bs[i]) for i in range(3)})
    xt = rp.from_numpy(x).to(device="cuda").requires_grad_(True)
    loss = net(xt).op_cross_entropy_loss(y.tolist())
    assert loss.shape == (1,)
    loss.backward()
    want = oracle.mlp_step(x, ws, bs, y, oracle.F32)
    t = 1e-5 * np.sqrt(784)
    assert abs(loss.sum_all() - float(want["loss"][0])) <= 1e-5 * float(want["loss"][0])
    assert oracle.rel_err(host(xt.grad), want["dX"]) <= t
    for i in range(3):
        fc = getattr(net, f"fc{i + 1}")
        assert oracle.rel_err(host(fc.weight.grad), want["dW"][i]) <= t
        assert oracle.rel_err(host(fc.bias.grad), want["db"][i]) <= t
    with pytest.raises(RuntimeError):
        net(xt).op_cross_entropy_loss([10] * batch)        # out-of-range target (reference ops/ops.c:5547-5549)


# ---- benchmark configuration 4 shape (scaled down) through the Python API: batched matmul on a permuted view, forward + backward
@pytest.mark.parametrize("dtype,tol", [("float64", 1e-11), ("float32", 2e-5), ("bfloat16", 4e-2)])
def test_attention_batched_matmul_on_permuted_view(dtype, tol):
    import torch
    rng = np.random.default_rng(53)
    B, H, S, D = 2, 3, 64, 32
    q, k, v, do = (rng.normal(0, 1, (B, H, S, D)) for _ in range(4))
    qt, kt, vt = (dev(a, dtype, grad=True) for a in (q, k, v))
    kT = kt.permute([0, 1, 3, 2])
    assert kT.shape == (B, H, D, S) and not kT.is_contiguous
    s = qt.op_matmul(kT)
    assert s.shape == (B, H, S, S)
    o = s.op_mul_scalar(1.0 / np.sqrt(D)).op_softmax(dim=-1).op_matmul(vt)
    assert o.shape == (B, H, S, D) and o.dtype == dtype
    # scalar loss: every entry of O_flat · W_flatᵀ summed, with random weights W so that all of dO is exercised
    w = dev(do, dtype)
    flat_o = o.reshape([B * H * S, D]); flat_w = w.reshape([B * H * S, D])
    loss = flat_o.op_matmul(flat_w.transpose(0, 1))          # [N, N]
    tq, tk, tv = (torch.tensor(host(t), requires_grad=True) for t in (qt, kt, vt))
    to = torch.softmax(tq @ tk.transpose(2, 3) / np.sqrt(D), -1) @ tv
    np.testing.assert_allclose(host(o), to.detach().numpy(), rtol=tol * 5, atol=tol)
    tw = torch.tensor(host(w))
    (to.reshape(-1, D) @ tw.reshape(-1, D).T).sum().backward()
    loss.op_sum_all().backward()
    for got, want in ((qt, tq), (kt, tk), (vt, tv)):
        assert got.grad.shape == (B, H, S, D)
        assert oracle.rel_err(host(got.grad), want.grad.numpy()) <= tol


# ---- the fused extension: one call for softmax(scale·q·kᵀ)·v, gradients through the fused backward
@pytest.mark.parametrize("dtype,tol", [("bfloat16", 4e-2), ("float16", 6e-3), ("float32", 2e-5)])
def test_fused_attention_op_matches_the_unfused_chain_and_torch(dtype, tol):
    import torch
    rng = np.random.default_rng(54)
    B, H, S, D = 2, 3, 96, 64
    q, k, v, do = (rng.normal(0, 1, (B, H, S, D)) for _ in range(4))
    qt, kt, vt = (dev(a, dtype, grad=True) for a in (q, k, v))
    scale = 1.0 / np.sqrt(D)
    o = qt.op_attention(kt, vt, scale)
    assert o.shape == (B, H, S, D) and o.dtype == dtype and o.requires_grad
    w = dev(do, dtype)
    o.reshape([B * H * S, D]).op_matmul(w.reshape([B * H * S, D]).transpose(0, 1)).op_sum_all().backward()
    # the same through the four separate ops
    q2, k2, v2 = (dev(host(t), dtype, grad=True) for t in (qt, kt, vt))
    o2 = q2.op_matmul(k2.permute([0, 1, 3, 2])).op_mul_scalar(scale).op_softmax(dim=-1).op_matmul(v2)
    o2.reshape([B * H * S, D]).op_matmul(w.reshape([B * H * S, D]).transpose(0, 1)).op_sum_all().backward()
    assert oracle.rel_err(host(o), host(o2)) <= tol
    # and against float64 autograd
    tq, tk, tv = (torch.tensor(host(t), requires_grad=True) for t in (qt, kt, vt))
    to = torch.softmax(tq @ tk.transpose(2, 3) * scale, -1) @ tv
    (to.reshape(-1, D) @ torch.tensor(host(w)).reshape(-1, D).T).sum().backward()
    assert oracle.rel_err(host(o), to.detach().numpy()) <= tol
    for got, chain, want in ((qt, q2, tq), (kt, k2, tk), (vt, v2, tv)):
        assert got.grad.shape == (B, H, S, D)
        assert oracle.rel_err(host(got.grad), want.grad.numpy()) <= tol
        assert oracle.rel_err(host(got.grad), host(chain.grad)) <= tol
    with pytest.raises(RuntimeError, match="op_attention operation failed"):
        dev(q, "float64").op_attention(dev(k, "float64"), dev(v, "float64"), scale)      # no float64 kernels


# ---- reference tests/stress/stress_edge_cases.py:41-42, 193-198
def test_error_conventions():
    a = rp.zeros([2, 3], device="cuda"); b = rp.zeros([2, 3], device="cuda")
    with pytest.raises(RuntimeError, match="op_matmul operation failed"):
        a.op_matmul(b)                                                        # inner dimensions differ
    with pytest.raises(RuntimeError):
        a.op_matmul(rp.zeros([3, 2]))                                         # cuda @ cpu must raise, not crash
    with pytest.raises(RuntimeError):
        a.op_matmul(rp.zeros([3, 2], device="cuda", dtype="float64"))         # dtype mismatch
    with pytest.raises(RuntimeError):
        rp.zeros([1], device="cuda:7")                                        # invalid ordinal on a one-GPU box
    with pytest.raises(RuntimeError):
        rp.zeros([4], device="cuda").op_matmul(rp.zeros([4], device="cuda"))  # 1-D operands
    with pytest.raises(RuntimeError):
        a.op_add(rp.zeros([4, 3], device="cuda"))                             # not broadcastable


# ---- reference tests/integration/test_module.py:108-131 and tests/stress/stress_e2e.py:60-85
def _train(seed, steps=50, lr=0.5):
    rng = np.random.default_rng(seed)
    rp.manual_seed(seed)
    x = rng.normal(0, 1, (16, 8)).astype(np.float32)
    y = (x[:, 0] + x[:, 1] > 0).astype(int).tolist()
    net = MLP([8, 16, 2]).to(device="cuda")
    xt = rp.from_numpy(x).to(device="cuda")
    losses = []
    for _ in range(steps):
        net.zero_grad()
        loss = net(xt).op_cross_entropy_loss(y)
        loss.backward()
        losses.append(loss.sum_all())
        for p in net.parameters():                                            # plain SGD written with tensor ops
            p.copy_(p.op_add(p.grad.mul_scalar(-lr)))
            p.requires_grad_(True)
    return losses, [host(p) for p in net.parameters()]


def test_training_halves_the_loss_and_is_deterministic():
    losses, params = _train(5)
    assert losses[-1] < 0.5 * losses[0]
    losses2, params2 = _train(5)
    assert losses == losses2
    for p, q in zip(params, params2):
        assert np.array_equal(p, q)


# ---- the usual head split x.reshape(B, S, H, D).permute(0, 2, 1, 3): its leading dims do not collapse into one batch
# stride, so forward AND backward take a dense copy of that operand; both gradients must exist and match the oracle
@pytest.mark.parametrize("dtype,tol", [("float64", 1e-12), ("float32", 1e-5 * 8), ("bfloat16", 2e-2)])
def test_batched_matmul_backward_on_head_split_views(dtype, tol):
    rng = np.random.default_rng(57)
    B, S, H, D = 2, 48, 3, 32
    code = {"float64": oracle.F64, "float32": oracle.F32, "bfloat16": oracle.BF16}[dtype]
    xq, xk = (oracle.to_f64(oracle.to_storage(rng.normal(0, 1, (B, S, H * D)), code), code) for _ in range(2))
    dq = dev(xq, dtype, grad=True); dk = dev(xk, dtype, grad=True)
    q = dq.reshape([B, S, H, D]).permute([0, 2, 1, 3])                # strides (S*H*D, D, H*D, 1)
    kT = dk.reshape([B, S, H, D]).permute([0, 2, 3, 1])               # K^T per head, a view as well
    assert not q.is_contiguous and not kT.is_contiguous
    s = q.op_matmul(kT)
    assert s.shape == (B, H, S, S)
    s.backward()                                                       # upstream of ones
    # oracle: per (b, h) slice, the reference's CPU matmul and its backward GEMMs on dense copies
    q4 = xq.reshape(B, S, H, D).transpose(0, 2, 1, 3); k4 = xk.reshape(B, S, H, D).transpose(0, 2, 1, 3)
    want_s = np.zeros((B, H, S, S)); want_dq = np.zeros((B, H, S, D)); want_dkT = np.zeros((B, H, D, S))
    ones = oracle.to_storage(np.ones((S, S)), code)
    for b in range(B):
        for h in range(H):
            a_ = oracle.to_storage(q4[b, h], code); b_ = oracle.to_storage(np.ascontiguousarray(k4[b, h].T), code)
            want_s[b, h] = oracle.to_f64(oracle.matmul(a_, b_, code), code)
            da, db = oracle.matmul_backward(a_, b_, ones, code)
            want_dq[b, h] = oracle.to_f64(da, code); want_dkT[b, h] = oracle.to_f64(db, code)
    assert oracle.rel_err(host(s), want_s) <= tol
    assert dq.has_grad and dk.has_grad
    got_dq = host(dq.grad).reshape(B, S, H, D).transpose(0, 2, 1, 3)
    got_dkT = host(dk.grad).reshape(B, S, H, D).transpose(0, 2, 3, 1)
    assert oracle.rel_err(got_dq, want_dq) <= tol
    assert oracle.rel_err(got_dkT, want_dkT) <= tol


# ---- a GEMM that fails inside backward() must surface (reference python/tensor_python.c:400-414 raises
# "backward operation failed"); the failure is forced from the host, nothing faulty reaches the device
def test_failure_inside_backward_raises_and_leaves_no_stale_grad():
    a = dev(np.arange(6.0).reshape(2, 3), "float32", grad=True)
    b = dev(np.arange(12.0).reshape(3, 4), "float32", grad=True)
    s = a.op_matmul(b).op_sum_all()
    rp._fail_gemm_after(1)                      # the next GEMM the host layer issues is dA = dC . B^T
    try:
        with pytest.raises(RuntimeError, match="backward"):
            s.backward()
    finally:
        rp._fail_gemm_after(0)
    assert not a.has_grad                        # the failed gradient is absent, not stale
    assert b.has_grad                            # the walk went on: dB = A^T . dC was computed
    b.zero_grad()
    # the graph was freed all the same and the tensors stay usable
    s2 = a.op_matmul(b).op_sum_all()
    s2.backward()
    assert np.array_equal(host(a.grad), np.tile(np.arange(12.0).reshape(3, 4).sum(1), (2, 1)))
    assert np.array_equal(host(b.grad), np.tile(np.arange(6.0).reshape(2, 3).sum(0)[:, None], (1, 4)))


# ---- benchmark configuration 4 at full size through the drop-in tensors: Q, K, V [16, 12, 512, 64], K^T as the 4-D
# permuted view (reference ops/ops.c:8639-8697: shape and strides permuted, data shared), forward and backward.  The two
# leading dims collapse into one batch stride inside the host layer; nothing is copied.
@pytest.mark.parametrize("dtype,tol_gemm,tol_chain", [("bfloat16", 2e-2, 3e-2), ("float32", 1e-5 * np.sqrt(512), 1e-5 * np.sqrt(512))])
def test_config4_full_size_on_4d_permuted_view(dtype, tol_gemm, tol_chain):
    import torch
    rng = np.random.default_rng(3)
    B, H, S, D = 16, 12, 512, 64
    code = {"float32": oracle.F32, "bfloat16": oracle.BF16}[dtype]
    q, k, v = (oracle.to_f64(oracle.to_storage(rng.normal(0, 1, (B, H, S, D)), code), code) for _ in range(3))
    qt, kt, vt = (dev(a, dtype, grad=True) for a in (q, k, v))
    kT = kt.permute([0, 1, 3, 2])
    assert kT.shape == (B, H, D, S) and not kT.is_contiguous
    s = qt.op_matmul(kT)
    assert s.shape == (B, H, S, S)
    # S alone against float64 at one GEMM's tolerance
    assert oracle.rel_err(host(s), np.matmul(q, k.transpose(0, 1, 3, 2))) <= tol_gemm
    o = s.op_mul_scalar(0.125).op_softmax(dim=-1).op_matmul(vt)
    assert o.shape == (B, H, S, D) and o.dtype == dtype
    o.backward()                                     # upstream of ones (reference core/tensor.c:223-228)
    for t in (qt, kt, vt):
        assert t.has_grad and t.grad.shape == (B, H, S, D)
    # the whole chain against float64 autograd
    tq, tk, tv = (torch.tensor(x, requires_grad=True) for x in (q, k, v))
    to = torch.softmax(tq @ tk.transpose(2, 3) * 0.125, -1) @ tv
    to.sum().backward()
    assert oracle.rel_err(host(o), to.detach().numpy()) <= tol_chain
    grads = {"dQ": host(qt.grad), "dK": host(kt.grad), "dV": host(vt.grad)}
    for name, want in (("dQ", tq.grad), ("dK", tk.grad), ("dV", tv.grad)):
        assert oracle.rel_err(grads[name], want.numpy()) <= tol_chain, name
    # and the CPU oracle (the reference's op chain, one rounding per op) on two (batch, head) slices
    ones = oracle.to_storage(np.ones((S, D)), code)
    o_host = host(o)
    for b, h in ((0, 0), (B - 1, H - 1)):
        want = oracle.attention(oracle.to_storage(q[b, h], code), oracle.to_storage(k[b, h], code), oracle.to_storage(v[b, h], code), code, scale=0.125, d_out=ones)
        assert oracle.rel_err(o_host[b, h], oracle.to_f64(want["O"], code)) <= tol_gemm, (b, h)
        for name in ("dQ", "dK", "dV"):
            assert oracle.rel_err(grads[name][b, h], oracle.to_f64(want[name], code)) <= tol_gemm, (name, b, h)


# ---- op_cross_entropy_loss with every reduction, on logits and on the output of op_softmax (which the op detects and
# treats as probabilities, reference ops/ops.c:5553-5585), and op_log_softmax with its backward (ops/ops.c:5693-5719,
# 5790-5860): values and gradients against torch in float64
@pytest.mark.parametrize("dtype,tol", [("float32", 4e-6), ("float64", 1e-12)])
@pytest.mark.parametrize("reduction", ["none", "sum", "mean"])
def test_cross_entropy_reductions_and_probability_inputs(dtype, tol, reduction):
    import torch
    rng = np.random.default_rng(58)
    batch, classes = 48, 10
    x = rng.normal(0, 2, (batch, classes)); w = rng.normal(0, 1, batch)
    targets = rng.integers(0, classes, batch).tolist()
    for through_softmax in (False, True):
        xt = dev(x, dtype, grad=True)
        src = xt.op_softmax(dim=-1) if through_softmax else xt
        loss = src.op_cross_entropy_loss(targets, reduction=reduction)
        assert loss.shape == ((batch,) if reduction == "none" else (1,))
        tx = torch.tensor(host(xt), requires_grad=True)
        tl = torch.nn.functional.cross_entropy(tx, torch.tensor(targets), reduction=reduction)
        np.testing.assert_allclose(host(loss), tl.detach().numpy().reshape(loss.shape), rtol=tol * 10, atol=tol)
        if reduction == "none":                       # weight the rows so that the per-row upstream gradient is exercised
            wt = dev(w.reshape(1, batch), dtype)
            wt.op_matmul(loss.reshape([batch, 1])).backward()
            (tl * torch.tensor(host(wt)[0])).sum().backward()
        else:
            loss.backward()
            tl.backward()
        assert oracle.rel_err(host(xt.grad), tx.grad.numpy()) <= tol * 20, (reduction, through_softmax)
    # explicit from_logits overrides the detection; an unknown reduction is refused
    xt = dev(x, dtype)
    a = xt.op_cross_entropy_loss(targets, reduction=reduction, from_logits=1)
    b = xt.op_cross_entropy_loss(targets, reduction=reduction)
    assert np.array_equal(host(a), host(b))
    with pytest.raises(ValueError):
        xt.op_cross_entropy_loss(targets, reduction="median")


@pytest.mark.parametrize("dtype,tol", [("float32", 4e-6), ("float64", 1e-12), ("bfloat16", 3e-2)])
def test_log_softmax_backward(dtype, tol):
    import torch
    rng = np.random.default_rng(59)
    x = rng.normal(0, 2, (6, 9, 5)); w = rng.normal(0, 1, (6, 9, 5))
    for dim in (-1, 1):
        xt = dev(x, dtype, grad=True)
        y = xt.op_log_softmax(dim=dim)
        assert y.requires_grad
        # loss = sum(y * w) written with the ops at hand: flatten and multiply by w as a column
        wt = dev(w.reshape(-1, 1), dtype)
        y.reshape([1, x.size]).op_matmul(wt).backward()
        tx = torch.tensor(host(xt), requires_grad=True)
        (torch.log_softmax(tx, dim) * torch.tensor(host(wt).reshape(x.shape))).sum().backward()
        np.testing.assert_allclose(host(y), torch.log_softmax(tx, dim).detach().numpy(), rtol=tol * 5, atol=tol * 5)
        assert oracle.rel_err(host(xt.grad), tx.grad.numpy()) <= tol * 10, dim


# ---- `x.op_mul_scalar(s).op_softmax()`: the scaled tensor is a temporary; forward and backward each run one pass less
@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_scaled_softmax_chain_with_and_without_a_held_intermediate(dtype):
    """The chained form never writes the scaled scores (its scalar multiply is still unlaunched when the softmax consumes
    it) and its backward hands the scores their gradient in one pass; with the intermediate held in a variable both stay
    two ops (reference ops/ops.c:6022-6086, 5721-5788).  Same bits either way, forward and backward, and the held
    intermediate reads back as the product."""
    rng = np.random.default_rng(33)
    s0 = rng.normal(0, 2, (6, 40, 64))
    up = rng.normal(0, 1, (6, 40, 64))

    def run(chained):
        s = dev(s0, dtype, grad=True)
        w = dev(up, dtype)
        if chained:
            p = s.op_mul_scalar(0.125).op_softmax()
            held = None
        else:
            held = s.op_mul_scalar(0.125)
            p = held.op_softmax()
        loss = p.op_matmul(w.transpose(1, 2)).op_sum_all()
        loss.backward()
        return host(p), host(s.grad), (host(held) if held is not None else None)

    p1, g1, _ = run(True)
    p2, g2, held = run(False)
    assert np.array_equal(p1, p2) and np.array_equal(g1, g2)
    assert np.array_equal(held, host(dev(s0, dtype).op_mul_scalar(0.125)))
    code = {"float32": oracle.F32, "bfloat16": oracle.BF16}[dtype]
    scaled = oracle.mul_scalar(oracle.to_storage(s0, code), 0.125, code)
    assert np.array_equal(held, oracle.to_f64(scaled, code))
    want = oracle.to_f64(oracle.softmax(scaled, code), code)
    assert oracle.rel_err(p1, want) <= (2e-6 if dtype == "float32" else 1.6e-2)
    # a temporary that other work touches before the softmax is materialised like any other tensor
    s = dev(s0, dtype)
    t = s.op_mul_scalar(0.125)
    u = t.op_relu()
    assert np.array_equal(host(u), np.maximum(host(t), 0.0))
