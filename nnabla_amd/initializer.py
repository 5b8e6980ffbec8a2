"""Parameter initializers with nnabla's names (python/src/nnabla/initializer.py): callables shape -> numpy array."""
import numpy as np

from . import random


class BaseInitializer(object):
    def __call__(self, shape):
        raise NotImplementedError()


class ConstantInitializer(BaseInitializer):
    def __init__(self, value=0):
        self.value = value

    def __call__(self, shape):
        return np.ones(shape, dtype=np.float32) * self.value


class UniformInitializer(BaseInitializer):
    def __init__(self, lim=(-1, 1), rng=None):
        self.rng = random.prng if rng is None else rng
        self.lim = lim

    def __call__(self, shape):
        return self.rng.uniform(self.lim[0], self.lim[1], size=shape).astype(np.float32)


class NormalInitializer(BaseInitializer):
    def __init__(self, sigma=1.0, rng=None):
        self.rng = random.prng if rng is None else rng
        self.sigma = sigma

    def __call__(self, shape):
        return (self.rng.randn(*shape) * self.sigma).astype(np.float32)


def calc_uniform_lim_glorot(inmaps, outmaps, kernel=(1, 1)):
    """Limits of Glorot's uniform initialization: sqrt(6 / (prod(kernel) * inmaps + outmaps))."""
    d = np.sqrt(6. / (np.prod(kernel) * inmaps + outmaps))
    return -d, d


def calc_normal_std_he_forward(inmaps, outmaps, kernel=(1, 1)):
    return np.sqrt(2. / (np.prod(kernel) * inmaps))


def calc_normal_std_glorot(inmaps, outmaps, kernel=(1, 1)):
    return np.sqrt(2. / (np.prod(kernel) * inmaps + outmaps))
