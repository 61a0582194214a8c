"""Which columns of a K-wide product the full-size tests compare element by element."""
import numpy as np


def sample_columns(K, seed):
    """One column inside every 32-column tile of the matrix-core kernels (at a different place in each tile), the first
    and the last column, and two drawn at random."""
    rng = np.random.default_rng(seed)
    cols = {0, K - 1}
    for t in range((K + 31) // 32):
        cols.add(min(K - 1, 32 * t + (7 * t + 3) % 32))
    cols.update(int(c) for c in rng.integers(0, K, 2))
    return sorted(cols)
