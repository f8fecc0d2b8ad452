"""YaRN rotary scaling: the per-pair frequency table and attention factor that the YaRN forms of the QK-norm + rotary
kernels read after eps in their `par` block. Host-side mirror of the reference's python/caminus/rope.py:27-50 (same
function names, arguments and results); the recipe is llama.cpp's rope_yarn / ggml_rope_yarn_corr_dims.

For pair j of n_rot / 2 (NeoX dims j and j + n_rot / 2):
    inv_j  = base ** (-2 j / n_rot)
    [lo, hi] = [floor(cd(beta_fast)), ceil(cd(beta_slow))] clipped to [0, n_rot - 1],
               cd(beta) = n_rot * ln(n_ctx_orig / (2 pi beta)) / (2 ln base)
    ramp_j = 1 - clip((j - lo) / max(0.001, hi - lo), 0, 1)
    freq_j = inv_j * (ramp_j + (1 - ramp_j) / factor)
    mscale = 1 + 0.1 ln(factor)   (factor <= 1: 1), applied to cos and sin
All in float64; the table is rounded to float32 once.
"""
import math

import numpy as np

BETA_FAST, BETA_SLOW = 32.0, 1.0
TABLE_FLOATS = 65            # freq[n_rot / 2] then mscale, for n_rot = 128


def corr_dims(n_rot, n_ctx_orig, base, beta_fast=BETA_FAST, beta_slow=BETA_SLOW):
    def cd(beta):
        return n_rot * math.log(n_ctx_orig / (beta * 2 * math.pi)) / (2 * math.log(base))
    return max(0.0, float(math.floor(cd(beta_fast)))), min(float(n_rot - 1), float(math.ceil(cd(beta_slow))))


def yarn_freqs(n_rot, base, factor, n_ctx_orig, beta_fast=BETA_FAST, beta_slow=BETA_SLOW):
    lo, hi = corr_dims(n_rot, n_ctx_orig, base, beta_fast, beta_slow)
    j = np.arange(n_rot // 2, dtype=np.float64)
    inv = base ** (-2.0 * j / n_rot)
    ramp = 1.0 - np.clip((j - lo) / max(0.001, hi - lo), 0.0, 1.0)
    return inv * (ramp + (1.0 - ramp) / factor)


def mscale(factor):
    return 1.0 if factor <= 1.0 else 1.0 + 0.1 * math.log(factor)


def yarn_table(n_rot, base, factor, n_ctx_orig):
    if n_rot != 128:
        raise ValueError(f'yarn_table: n_rot {n_rot} (the YaRN kernels are built for 128)')
    return np.concatenate([yarn_freqs(n_rot, base, factor, n_ctx_orig), [mscale(factor)]]).astype(np.float32)


class YarnMode:
    """factor and original context of a long-context mode, and the table it makes"""
    kind = 'yarn'

    def __init__(self, factor, n_ctx_orig):
        self.factor, self.n_ctx_orig = float(factor), int(n_ctx_orig)
        if not self.factor > 1.0 or self.n_ctx_orig < 1:
            raise ValueError(f'YaRN: factor {factor} (> 1), original context {n_ctx_orig}')

    @property
    def max_ctx(self):
        return int(self.factor * self.n_ctx_orig)

    def key(self):
        return f'yarn:{self.factor:g}:{self.n_ctx_orig}:{BETA_FAST:g}:{BETA_SLOW:g}'

    def table(self, n_rot, base):
        return yarn_table(n_rot, base, self.factor, self.n_ctx_orig)

    def __repr__(self):
        return f'YarnMode(x{self.factor:g} from {self.n_ctx_orig})'
