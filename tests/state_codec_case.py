"""States for the state codec's tests: the reference test's value classes (state_codec_metal_test.mm:88-177, :179-257)."""
import numpy as np


def running_state(rng, rows, columns):
    """Rows of mixed magnitudes; blocks whose largest magnitude lies in the first half, the second, both, or nowhere
    (zeros); tiny and huge finite blocks; a block of one value."""
    v = (rng.standard_normal((rows, columns)) * np.exp(rng.uniform(-6, 3, (rows, 1)))).astype(np.float32)
    flat = v.reshape(-1, 32)
    n = flat.shape[0]
    flat[0 % n] = 0
    flat[1 % n, :16] *= 100
    flat[2 % n, 16:] *= 100
    flat[3 % n, 3] = flat[3 % n, 19] = 7.5
    flat[4 % n] = np.float32(1e-39) * np.arange(-16, 16)            # subnormal values and scale
    flat[5 % n] = np.float32(3e38) * np.linspace(-1, 1, 32)          # near the largest finite
    flat[6 % n] = 0
    flat[6 % n, 31] = -2.5
    flat[7 % n] = np.float32(127.0) * np.linspace(-1, 1, 32)         # ties and exact codes
    flat[8 % n] = np.arange(32) - 15.5                               # halves: rint to even
    return flat.reshape(rows, columns)


def with_non_finite(state):
    """NaN in a block's first half, an infinity in another's second, -infinity in a third; their neighbours finite."""
    flat = state.copy().reshape(-1, 32)
    n = flat.shape[0]
    flat[10 % n, 5] = np.nan
    flat[12 % n, 20] = np.inf
    flat[14 % n, 0] = -np.inf
    return flat.reshape(state.shape)
