"""Row initialisers: the host-side mirror of ``recis.nn.initializers`` and of the
generator family behind it (csrc/embedding/initializer.h:15-66, initializer.cc:26-366).

An initialiser describes a distribution; ``build()`` turns it into a generator
that fills ``[rows, *embedding_shape]`` tensors with torch's RNG on the slot's
device. As in the reference, rows are drawn when storage is created (and drawn
again for rows freed by eviction), not per key.
"""
import math

import torch


def _f32(v):
    """The reference keeps every distribution parameter in a C++ ``float`` member
    (initializer.cc:59-60,82-83,122,...): the value the torch call sees is the rounded one."""
    return float(torch.tensor(float(v), dtype=torch.float32))


class _Generator:
    """Counterpart of ``torch.classes.recis.Generator``.

    ``generate(shape)`` fills a new tensor. Initialisers that depend on fan-in / fan-out take the
    fans from the generated tensor, as the reference does (``torch::nn::init::*`` on the block it
    has just allocated, initializer.cc:108-190): from ``shape`` when given (``Slot::GenVal`` for
    re-initialised rows, slot_group.cc:112-116), else from the generator's own ``[block_size, D]``
    shape. ``fan_shape`` overrides that for callers that allocate several blocks in one tensor."""

    def __init__(self, shape, dtype, fill, desc):
        self.shape = list(shape)
        self.dtype = dtype
        self.device = torch.device("cpu")
        # fill(tensor, torch generator[, fan shape]): initialisers that need no fans take two arguments
        import inspect
        self._fill = fill if len(inspect.signature(fill).parameters) >= 3 else (lambda t, g, fs: fill(t, g))
        self._desc = desc
        self.torch_generator = None

    def set_device(self, device):
        self.device = torch.device(device)
        g = self.torch_generator
        if g is not None and g.device.type != self.device.type:
            raise ValueError("the torch.Generator of %s lives on %s but the rows are drawn on %s: pass a generator "
                             "of the table's device" % (self._desc, g.device, self.device))

    def generate(self, shape=None, fan_shape=None):
        shape = list(self.shape if shape is None else shape)
        work = self.dtype if self.dtype.is_floating_point and self.dtype != torch.float16 \
            and self.dtype != torch.bfloat16 else (torch.float32 if self.dtype.is_floating_point else self.dtype)
        t = torch.empty(shape, dtype=work, device=self.device)
        if t.numel():
            self._fill(t, self.torch_generator, list(fan_shape if fan_shape is not None else shape))
        return t if work == self.dtype else t.to(self.dtype)

    def __str__(self):
        return self._desc


def _fans(shape):
    # [rows, D...]: fan_in / fan_out as torch.nn.init computes them for that tensor
    if len(shape) < 2:
        raise ValueError("fan in/out needs at least 2 dimensions")
    receptive = 1
    for d in shape[2:]:
        receptive *= d
    return shape[1] * receptive, shape[0] * receptive


class Initializer:
    def __init__(self):
        self._shape = None
        self._dtype = torch.float32
        self._impl = None

    def set_shape(self, shape):
        self._shape = list(shape)

    def set_dtype(self, dtype):
        self._dtype = dtype

    def build(self):
        # an instance can be built once (recis/nn/initializers.py:20-36)
        if self._impl is None:
            self._impl = self._build_impl()
        return self

    def impl(self):
        if self._impl is None:
            raise RuntimeError("initializer must be built before use")
        return self._impl

    def generate(self):
        return self.impl().generate()

    def _build_impl(self):
        raise NotImplementedError


class ConstantInitializer(Initializer):
    def __init__(self, init_val=0.0):
        super().__init__()
        self._init_val = init_val

    def _build_impl(self):
        v = _f32(self._init_val)
        return _Generator(self._shape, self._dtype, lambda t, g: t.fill_(v),
                          "ConstantInitializer(init_val=%s)" % self._init_val)

    def __str__(self):
        return "ConstantInitializer(init_val=%s)" % self._init_val


class UniformInitializer(Initializer):
    def __init__(self, a=0.0, b=1.0, generator=None):
        super().__init__()
        self._a, self._b, self._gen = a, b, generator

    def _build_impl(self):
        a, b = _f32(self._a), _f32(self._b)
        g = _Generator(self._shape, self._dtype, lambda t, gen: t.uniform_(a, b, generator=gen),
                       "UniformInitializer(a=%s, b=%s)" % (self._a, self._b))
        g.torch_generator = self._gen
        return g

    def __str__(self):
        return "UniformInitializer(a=%s, b=%s)" % (self._a, self._b)


class NormalInitializer(Initializer):
    def __init__(self, mean=0.0, std=1.0, generator=None):
        super().__init__()
        self._mean, self._std, self._gen = mean, std, generator

    def _build_impl(self):
        mean, std = _f32(self._mean), _f32(self._std)
        g = _Generator(self._shape, self._dtype, lambda t, gen: t.normal_(mean, std, generator=gen),
                       "NormalInitializer(mean=%s, std=%s)" % (self._mean, self._std))
        g.torch_generator = self._gen
        return g

    def __str__(self):
        return "NormalInitializer(mean=%s, std=%s)" % (self._mean, self._std)


class XavierUniformInitializer(Initializer):
    def __init__(self, gain=1.0, generator=None):
        super().__init__()
        self._gain, self._gen = gain, generator

    def _build_impl(self):
        gain = _f32(self._gain)

        def fill(t, gen, fan_shape):  # torch::nn::init::xavier_uniform_, in its order of operations
            fan_in, fan_out = _fans(fan_shape)
            bound = math.sqrt(3.0) * (gain * math.sqrt(2.0 / (fan_in + fan_out)))
            t.uniform_(-bound, bound, generator=gen)

        g = _Generator(self._shape, self._dtype, fill, str(self))
        g.torch_generator = self._gen
        return g

    def __str__(self):
        return "XavierUniformInitializer(gain=%s)" % self._gain


class XavierNormalInitializer(Initializer):
    def __init__(self, gain=1.0, generator=None):
        super().__init__()
        self._gain, self._gen = gain, generator

    def _build_impl(self):
        gain = _f32(self._gain)

        def fill(t, gen, fan_shape):  # torch::nn::init::xavier_normal_
            fan_in, fan_out = _fans(fan_shape)
            t.normal_(0.0, gain * math.sqrt(2.0 / (fan_in + fan_out)), generator=gen)

        g = _Generator(self._shape, self._dtype, fill, str(self))
        g.torch_generator = self._gen
        return g

    def __str__(self):
        return "XavierNormalInitializer(gain=%s)" % self._gain


class KaimingUniformInitializer(Initializer):
    def __init__(self, a=0.0, mode="fan_in", nonlinearity="leaky_relu", generator=None):
        super().__init__()
        self._a, self._mode, self._nl, self._gen = a, mode, nonlinearity, generator

    def _bound(self, fan_shape):
        # torch::nn::init::kaiming_uniform_, in its order of operations
        fan_in, fan_out = _fans(fan_shape)
        fan = fan_in if self._mode == "fan_in" else fan_out
        gain = torch.nn.init.calculate_gain(self._nl, _f32(self._a))
        return math.sqrt(3.0) * (gain / math.sqrt(fan))

    def _build_impl(self):
        if self._mode not in ("fan_in", "fan_out"):
            raise ValueError("%s not in [fan_in, fan_out]" % self._mode)

        def fill(t, gen, fan_shape):
            bound = self._bound(fan_shape)
            t.uniform_(-bound, bound, generator=gen)

        g = _Generator(self._shape, self._dtype, fill, str(self))
        g.torch_generator = self._gen
        return g

    def __str__(self):
        return "%s(a=%s, mode=%s, nonlinearity=%s)" % (type(self).__name__, self._a, self._mode, self._nl)


class KaimingNormalInitializer(KaimingUniformInitializer):
    """The reference builds the *uniform* generator for this class too
    (recis/nn/initializers.py:585); kept as is."""


class TruncNormalInitializer(Initializer):
    def __init__(self, mean=0.0, std=1.0, a=-2.0, b=2.0, generator=None):
        super().__init__()
        self._mean, self._std, self._a, self._b, self._gen = mean, std, a, b, generator

    def _build_impl(self):
        mean, std, a, b = _f32(self._mean), _f32(self._std), _f32(self._a), _f32(self._b)

        def fill(t, gen, fan_shape):
            # inverse-CDF sampling between absolute bounds a and b (initializer.cc:216-229); the
            # reference does the bound arithmetic in C++ float: every step is rounded the same way here
            def ncdf(x):
                return _f32((1.0 + math.erf(x / math.sqrt(2.0))) / 2.0)
            lo, hi = ncdf(_f32(_f32(a - mean) / std)), ncdf(_f32(_f32(b - mean) / std))
            t.uniform_(_f32(_f32(2 * lo) - 1), _f32(_f32(2 * hi) - 1), generator=gen)
            t.erfinv_().mul_(std * math.sqrt(2.0)).add_(mean).clamp_(min=a, max=b)

        g = _Generator(self._shape, self._dtype, fill, str(self))
        g.torch_generator = self._gen
        return g

    def __str__(self):
        return "TruncNormalInitializer(mean=%s, std=%s, a=%s, b=%s)" % (self._mean, self._std, self._a, self._b)
