"""Parameter bookkeeping (`Module`), the affine layer (`Linear`), the convolution layer (`Conv2d`) and the
recurrent cells (`LSTMCell`, `GRUCell`).

Behaviour kept from the reference's recpulse/module.py:
  * a module records its parameters in `tracked` under their attribute names; assigning a
    child module copies the child's entries under dotted names ("fc1.weight") and lists the
    child (and its own children) in `_modules` (reference :14-26);
  * `parameters()` is the tracked tensors that require grad (:37-44);
  * `to()` moves every tracked tensor in place and re-arms requires_grad (:46-60);
  * `load_state()` copies by name and ignores unknown names (:62-71);
  * `Linear` stores its weight as [in_features, out_features] (not transposed), initialised
    N(0, 1/in_features), bias zeros (:91-108), and computes x·W then + bias (:110-114).
  * `Conv2d` stores its weight as [out_channels, in_channels, kH, kW], initialised
    N(0, 1/(in_channels*kH*kW)), bias zeros, and accepts ints or pairs for kernel size, stride,
    padding and dilation (:117-155).
  * `LSTMCell` / `GRUCell` store weight_ih [input_size, G*hidden] and weight_hh [hidden, G*hidden] (G = 4: i, f, g,
    o; G = 3: r, z, n), initialised N(0, 1/hidden), biases zeros; a missing state is zeros; LSTMCell returns
    (h_next, c_next), GRUCell h_next (:255-351).  A step here is one autograd node (two GEMMs and one fused
    element-wise kernel) instead of the reference's twenty-odd ops.
The Linear forward pass issues ONE launch (GEMM with the bias add in its epilogue) through
`Tensor.op_linear`; the two-op form the reference uses gives the same values and is kept as
`forward_two_ops` for comparison.
"""
import math

import recpulse_cuda as rp


def _is_private(name):
    return name == "tracked" or name.startswith("_")


class Module:
    def __init__(self):
        self.tracked = {}
        self._modules = {}
        self._training = True

    # -- registration ---------------------------------------------------------------
    def track(self, name, tensor):
        """Record `tensor` as a parameter (or buffer) called `name`; returns the tensor."""
        self.tracked[name] = tensor
        return tensor

    def __setattr__(self, name, value):
        if not _is_private(name) and isinstance(value, Module):
            self._adopt(name, value)
        object.__setattr__(self, name, value)

    def _adopt(self, name, child):
        self._modules[name] = child
        self.tracked.update({f"{name}.{key}": tensor for key, tensor in child.tracked.items()})
        self._modules.update({f"{name}.{key}": sub for key, sub in child._modules.items()})

    # -- calling ----------------------------------------------------------------------
    def forward(self, *args, **kwargs):
        raise NotImplementedError(f"{type(self).__name__} does not define forward()")

    def __call__(self, *args, **kwargs):
        return self.forward(*args, **kwargs)

    def keep(self, tensor):
        return tensor

    # -- views of the parameters -------------------------------------------------------
    def learnable(self):
        return {name: t for name, t in self.tracked.items() if t.requires_grad}

    def frozen(self):
        return {name: t for name, t in self.tracked.items() if not t.requires_grad}

    def parameters(self):
        return list(self.learnable().values())

    def zero_grad(self):
        for tensor in self.parameters():
            tensor.zero_grad()

    # -- placement and state -----------------------------------------------------------
    def to(self, device=None, dtype=None):
        where = {key: val for key, val in (("device", device), ("dtype", dtype)) if val is not None}
        if where:
            for tensor in self.tracked.values():
                wanted_grad = tensor.requires_grad
                tensor.to(inplace=True, **where)
                if wanted_grad:
                    tensor.requires_grad_(True)
        return self

    def load_state(self, state_dict):
        for name in state_dict.keys() & self.tracked.keys():
            target = self.tracked[name]
            wanted_grad = target.requires_grad
            target.copy_(state_dict[name])
            if wanted_grad:
                target.requires_grad_(True)

    def state(self):
        return dict(self.tracked)

    def train(self):
        return self._set_mode(True)

    def eval(self):
        return self._set_mode(False)

    def _set_mode(self, training):
        self._training = training
        for child in self._modules.values():
            child._set_mode(training)
        return self


class Linear(Module):
    """y = x · W + b with W of shape [in_features, out_features]."""

    def __init__(self, in_features, out_features, bias=True):
        super().__init__()
        self.in_features, self.out_features = in_features, out_features
        init = rp.randn([in_features, out_features]).mul_scalar(1.0 / math.sqrt(in_features))
        self.weight = self.track("weight", init.requires_grad_(True))
        self.bias = self.track("bias", rp.zeros([out_features]).requires_grad_(True)) if bias else None

    def forward(self, x):
        return self.keep(x.op_linear(self.weight, self.bias))

    def forward_two_ops(self, x):
        out = self.keep(x.op_matmul(self.weight))
        return out if self.bias is None else self.keep(out.op_add(self.bias))


def _pair(value):
    return (value, value) if isinstance(value, int) else tuple(value)


class Conv2d(Module):
    """y = conv2d(x, W) + b over x [N, in_channels, H, W] with W [out_channels, in_channels, kH, kW]."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1, bias=True):
        super().__init__()
        self.in_channels, self.out_channels = in_channels, out_channels
        self.kernel_size, self.stride, self.padding, self.dilation = _pair(kernel_size), _pair(stride), _pair(padding), _pair(dilation)
        kh, kw = self.kernel_size
        fan_in = in_channels * kh * kw
        init = rp.randn([out_channels, in_channels, kh, kw]).mul_scalar(1.0 / math.sqrt(fan_in))
        self.weight = self.track("weight", init.requires_grad_(True))
        self.bias = self.track("bias", rp.zeros([out_channels]).requires_grad_(True)) if bias else None

    def forward(self, x):
        return self.keep(x.op_conv2d(self.weight, bias=self.bias, stride_h=self.stride[0], stride_w=self.stride[1],
                                     pad_h=self.padding[0], pad_w=self.padding[1],
                                     dilation_h=self.dilation[0], dilation_w=self.dilation[1]))


class _RecurrentCell(Module):
    GATES = 0

    def __init__(self, input_size, hidden_size, bias=True):
        super().__init__()
        self.input_size, self.hidden_size = input_size, hidden_size
        scale = 1.0 / math.sqrt(hidden_size)
        g = self.GATES * hidden_size
        self.weight_ih = self.track("weight_ih", rp.randn([input_size, g]).mul_scalar(scale).requires_grad_(True))
        self.weight_hh = self.track("weight_hh", rp.randn([hidden_size, g]).mul_scalar(scale).requires_grad_(True))
        self.bias_ih = self.track("bias_ih", rp.zeros([g]).requires_grad_(True)) if bias else None
        self.bias_hh = self.track("bias_hh", rp.zeros([g]).requires_grad_(True)) if bias else None

    def _zero_state(self, x):
        return rp.zeros([x.shape[0], self.hidden_size], dtype=x.dtype, device=str(x.device))


class LSTMCell(_RecurrentCell):
    """(h_next, c_next) = LSTM step of x [B, input_size] from state (h, c), gates in the order i, f, g, o."""
    GATES = 4

    def forward(self, x, state=None):
        h, c = state if state is not None else (self._zero_state(x), self._zero_state(x))
        hc = self.keep(x.op_lstm_cell(h, c, self.weight_ih, self.weight_hh, self.bias_ih, self.bias_hh))
        batch, hid = x.shape[0], self.hidden_size
        return self.keep(hc.slice([0, 0], [batch, hid])), self.keep(hc.slice([0, hid], [batch, 2 * hid]))


class GRUCell(_RecurrentCell):
    """h_next = GRU step of x [B, input_size] from h, gates in the order r, z, n."""
    GATES = 3

    def forward(self, x, h=None):
        h = h if h is not None else self._zero_state(x)
        return self.keep(x.op_gru_cell(h, self.weight_ih, self.weight_hh, self.bias_ih, self.bias_hh))

