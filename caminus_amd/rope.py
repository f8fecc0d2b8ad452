"""YaRN rotary tables for the QK-norm + rotary kernels.

The YaRN forms of camx_q3p_qk_rope / camx_q3p_qk_rope_q8 / camx_qk_rope_bf16 / camx_qk_rope_paged read 65 extra floats
after `eps` in their parameter block: one angular frequency per rotary pair, then the factor that multiplies cos and sin.
This module makes that block on the host. It offers the reference's names (python/caminus/rope.py:27-50 yarn_freqs,
mscale, yarn_table; :53-74 YarnMode) with the same arguments and the same float32 results.

Arithmetic (float64 throughout, one rounding to float32 at the end). With P = n_rot / 2 pairs, pair j rotates NeoX dims
j and j + P:
    extrapolated frequency  e_j = base ** (-2 j / n_rot)                      (what plain rotary uses)
    interpolated frequency  e_j / factor                                      (positions squeezed into the trained range)
    blend                   freq_j = e_j * (keep_j + (1 - keep_j) / factor)
    keep_j = 1 - clip((j - lo) / max(0.001, hi - lo), 0, 1)
    lo = max(0, floor(turns(beta_fast))),  hi = min(n_rot - 1, ceil(turns(beta_slow)))
    turns(beta) = n_rot * ln(n_ctx_orig / (2 pi beta)) / (2 ln base)          (the pair that makes beta turns over the
                                                                               original context)
    attention factor        1 + 0.1 ln(factor) for factor > 1, else 1
For n_rot 128, base 1e6, factor 4, original context 32768: lo, hi = 23, 40; pairs below 23 keep e_j, pairs from 40 up use
e_j / 4, and the factor is 1.1386294 in float32.
"""
import math
from dataclasses import dataclass

import numpy as np

BETA_FAST = 32.0
BETA_SLOW = 1.0
TABLE_FLOATS = 65            # 64 pair frequencies + the attention factor (head dim 128)
_KERNEL_N_ROT = 128          # the YaRN kernels rotate whole 128-wide heads


def _turns_dim(beta, n_rot, n_ctx_orig, base):
    return n_rot * math.log(n_ctx_orig / (beta * 2 * math.pi)) / (2 * math.log(base))


def corr_dims(n_rot, n_ctx_orig, base, beta_fast=BETA_FAST, beta_slow=BETA_SLOW):
    """(lo, hi) as floats: the pairs between which the blend ramps from keep to interpolate"""
    lo = float(math.floor(_turns_dim(beta_fast, n_rot, n_ctx_orig, base)))
    hi = float(math.ceil(_turns_dim(beta_slow, n_rot, n_ctx_orig, base)))
    return max(0.0, lo), min(float(n_rot - 1), hi)


def yarn_freqs(n_rot, base, factor, n_ctx_orig, beta_fast=BETA_FAST, beta_slow=BETA_SLOW):
    """float64 [n_rot / 2]: the angle of pair j at position p is p * freq[j]"""
    lo, hi = corr_dims(n_rot, n_ctx_orig, base, beta_fast, beta_slow)
    pair = np.arange(n_rot // 2, dtype=np.float64)
    extrap = base ** (-2.0 * pair / n_rot)
    keep = 1.0 - np.clip((pair - lo) / max(0.001, hi - lo), 0.0, 1.0)
    return extrap * (keep + (1.0 - keep) / factor)


def mscale(factor):
    return 1.0 + 0.1 * math.log(factor) if factor > 1.0 else 1.0


def yarn_table(n_rot, base, factor, n_ctx_orig):
    """float32 [TABLE_FLOATS] = freq | mscale, laid out as the kernels read it"""
    if n_rot != _KERNEL_N_ROT:
        raise ValueError(f'yarn_table: n_rot {n_rot} (the YaRN kernels are built for 128)')
    out = np.empty(TABLE_FLOATS, dtype=np.float64)
    out[:-1] = yarn_freqs(n_rot, base, factor, n_ctx_orig)
    out[-1] = mscale(factor)
    return out.astype(np.float32)


@dataclass(init=False, repr=False)
class YarnMode:
    """A long-context rotary mode: scaling factor and the context length the model was trained at."""
    factor: float
    n_ctx_orig: int
    kind = 'yarn'

    def __init__(self, factor, n_ctx_orig):
        f, n = float(factor), int(n_ctx_orig)
        if not f > 1.0 or n < 1:
            raise ValueError(f'YaRN: factor {factor} (> 1), original context {n_ctx_orig}')
        self.factor, self.n_ctx_orig = f, n

    @property
    def max_ctx(self):
        return int(self.factor * self.n_ctx_orig)

    def key(self):
        """a string that differs whenever the table would"""
        return ':'.join(['yarn', f'{self.factor:g}', str(self.n_ctx_orig), f'{BETA_FAST:g}', f'{BETA_SLOW:g}'])

    def table(self, n_rot, base):
        return yarn_table(n_rot, base, self.factor, self.n_ctx_orig)

    def __repr__(self):
        return f'YarnMode(x{self.factor:g} from {self.n_ctx_orig})'
