"""The process-wide pseudo random generator of the initializers (python/src/nnabla/random.py: seed 313)."""
import numpy as np

prng = np.random.RandomState(313)


def seed(seed_value):
    global prng
    prng = np.random.RandomState(seed_value)


def set_function_seed(seed_value):
    seed(seed_value)
