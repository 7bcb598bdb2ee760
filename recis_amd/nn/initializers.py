"""Row initialisers: the host-side mirror of ``recis.nn.initializers`` and of the
generator family behind it (csrc/embedding/initializer.h:15-66, initializer.cc:26-366).

An initialiser describes a distribution; ``build()`` turns it into a generator
that fills ``[rows, *embedding_shape]`` tensors with torch's RNG on the slot's
device. As in the reference, rows are drawn when storage is created (and drawn
again for rows freed by eviction), not per key.
"""
import torch


def _gen():
    """``torch.classes.recis.Generator``: the generator family lives in recis.so
    (recis_amd/csrc/torch/table.cc), as the reference's lives in its library."""
    from .. import torch_library
    torch_library.load()
    return torch.classes.recis.Generator


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
        return _gen().generate(self.impl())

    def _build_impl(self):
        raise NotImplementedError


class ConstantInitializer(Initializer):
    def __init__(self, init_val=0.0):
        super().__init__()
        self._init_val = init_val

    def _build_impl(self):
        return _gen().make_constant_generator(self._shape, self._dtype, float(self._init_val))

    def __str__(self):
        return "ConstantInitializer(init_val=%s)" % self._init_val


class UniformInitializer(Initializer):
    def __init__(self, a=0.0, b=1.0, generator=None):
        super().__init__()
        self._a, self._b, self._gen = a, b, generator

    def _build_impl(self):
        return _gen().make_uniform_generator(self._shape, self._dtype, float(self._a), float(self._b), self._gen)

    def __str__(self):
        return "UniformInitializer(a=%s, b=%s)" % (self._a, self._b)


class NormalInitializer(Initializer):
    def __init__(self, mean=0.0, std=1.0, generator=None):
        super().__init__()
        self._mean, self._std, self._gen = mean, std, generator

    def _build_impl(self):
        return _gen().make_normal_generator(self._shape, self._dtype, float(self._mean), float(self._std), self._gen)

    def __str__(self):
        return "NormalInitializer(mean=%s, std=%s)" % (self._mean, self._std)


class XavierUniformInitializer(Initializer):
    def __init__(self, gain=1.0, generator=None):
        super().__init__()
        self._gain, self._gen = gain, generator

    def _build_impl(self):
        return _gen().make_xavier_uniform_generator(self._shape, self._dtype, float(self._gain), self._gen)

    def __str__(self):
        return "XavierUniformInitializer(gain=%s)" % self._gain


class XavierNormalInitializer(Initializer):
    def __init__(self, gain=1.0, generator=None):
        super().__init__()
        self._gain, self._gen = gain, generator

    def _build_impl(self):
        return _gen().make_xavier_normal_generator(self._shape, self._dtype, float(self._gain), self._gen)

    def __str__(self):
        return "XavierNormalInitializer(gain=%s)" % self._gain


class KaimingUniformInitializer(Initializer):
    def __init__(self, a=0.0, mode="fan_in", nonlinearity="leaky_relu", generator=None):
        super().__init__()
        self._a, self._mode, self._nl, self._gen = a, mode, nonlinearity, generator

    def _build_impl(self):
        if self._mode not in ("fan_in", "fan_out"):
            raise ValueError("%s not in [fan_in, fan_out]" % self._mode)
        return _gen().make_kaiming_uniform_generator(self._shape, self._dtype, float(self._a), self._mode, self._nl,
                                                     self._gen)

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
        return _gen().make_trunc_normal_generator(self._shape, self._dtype, float(self._mean), float(self._std),
                                                  float(self._a), float(self._b), self._gen)

    def __str__(self):
        return "TruncNormalInitializer(mean=%s, std=%s, a=%s, b=%s)" % (self._mean, self._std, self._a, self._b)


class TensorInitializer(Initializer):
    """Rows taken from a given ``[rows, D]`` tensor, in order, starting over at its end (an addition:
    the reference has no such generator). For tables that start from rows the caller already has."""

    def __init__(self, source):
        super().__init__()
        self._source = source

    def _build_impl(self):
        return _gen().make_tensor_generator(self._shape, self._dtype, self._source)

    def __str__(self):
        return "TensorInitializer(rows=%d)" % self._source.shape[0]
