"""Launch the row kernels from a PyTorch process through the reference's own launcher surface.

The reference loads gfx1100 code objects and launches their `extern "C"` kernels with
`Module(name).<symbol>(grid, block, *args, shmem=0, stream=None)` (python/caminus/device/hip.py:77-123). Here the same
call reaches libcamx.so's C ABI (include/camx.h): `Module(name)` accepts the reference's code-object names whose kernels
this library provides, attribute lookup accepts the reference's symbol names, arguments keep their order and types
(tensors become device pointers, scalars are explicit ctypes values, None-pointers are c_void_p(None)), the launch goes
to torch's current stream, and errors surface as the same RuntimeError text. What differs, by design: the library picks
its own launch geometry for gfx950, so `grid` and `block` only tell how many rows / tokens / elements the call covers
(a reference kernel that takes its extent from the grid gets it passed explicitly), and they are checked against the
shape arguments where the reference kernel would have read them.

There is no fallback path: a missing library is a FileNotFoundError, an unknown symbol an AttributeError.
"""
import ctypes

import torch

from . import kernels as _kernels
from . import lib as _lib

# set by a graph recorder while a chunk is captured or patched (None: launches go straight through); see Kernel.__call__
RECORD = None
BUILD, BUILD_FROM = _kernels.kernel_dir()
LOADED = []          # module names this process loaded, in order

I, F, L64 = ctypes.c_int, ctypes.c_float, ctypes.c_int64


def hip():
    """the loaded C-ABI library (the counterpart of the reference's libamdhip64 handle)"""
    if not getattr(torch.version, 'hip', None):
        raise RuntimeError('caminus_amd.device.hip needs a ROCm build of PyTorch')
    return _lib.load()


def check(err):
    if err != 0:
        raise RuntimeError(f'HIP error {err}: {_lib.load().camx_error_string(int(err)).decode()}')


def _val(a):
    return a.value if hasattr(a, 'value') else a


def _ceil(a, b):
    return -(-int(a) // int(b))


# ---- symbol table: reference symbol -> (C entry point, adapter(grid, block, vals) -> C argument list) -----------------------
# vals are the launch arguments after tensor -> c_void_p conversion, in the reference kernel's order.

def _plain(name):
    return name, lambda g, b, v: list(v)


def _rows(name):
    """the reference kernel runs one workgroup per row / token: the row count is grid[0]"""
    return name, lambda g, b, v: list(v) + [I(g[0])]


def _expect(cond, what):
    if not cond:
        raise ValueError(f'launch geometry does not match its arguments: {what}')


def _gg_q8_1(g, b, v):           # gg_quantize_q8_1(x, y, n): one thread per value
    n = _val(v[2])
    _expect(g[0] * b[0] >= n, f'gg_quantize_q8_1 covers {g[0] * b[0]} < n {n}')
    return [v[0], v[1], L64(n), I(0), F(0.0), ctypes.c_void_p(None)]


def _qk_rope(yarn, q8):
    def ad(g, b, v):             # (qkv, ldq, nh, nkv, par, pos0, q16, cache[, err]); grid (n, nh + nkv)
        _expect(g[1] == _val(v[2]) + _val(v[3]), f'q3p_qk_rope grid.y {g[1]} != nh + nkv')
        return list(v) + [I(g[0]), I(int(yarn))]
    return ('camx_q3p_qk_rope_q8' if q8 else 'camx_q3p_qk_rope'), ad


def _pf_qk_nr(g, b, v):          # (xin, head_stride, heads, w, D, nrot, theta_scale, eps, pos0, out); grid T * heads
    heads = _val(v[2])
    _expect(g[0] % heads == 0, f'pf_qk_nr grid {g[0]} is not a multiple of heads {heads}')
    return list(v) + [I(g[0] // heads), I(0)]


def _pf_gdn_l2(g, b, v):         # (x, y, heads, K, ldx, rs); grid T * heads
    heads = _val(v[2])
    _expect(g[0] % heads == 0, f'pf_gdn_l2 grid {g[0]} is not a multiple of heads {heads}')
    return list(v) + [I(g[0] // heads), I(0)]


def _pf_rms_mul(K):
    return 'camx_pf_rms_mul', lambda g, b, v: list(v) + [I(K)]


def _gate(io):
    return 'camx_gate_mul', lambda g, b, v: [v[0], v[1], v[2], L64(_val(v[3])), v[4], v[5], v[6], I(io)]


def _actq(is_bf16, codes):
    def ad(g, b, v):             # (x, y, s, [codes,] K, clip, qmax); grid M
        if codes: x, y, s, c, K, clip, qmax = v
        else: (x, y, s, K, clip, qmax), c = v, ctypes.c_void_p(None)
        return [x, I(int(is_bf16)), y, s, c, K, clip, qmax, I(g[0])]
    return 'camx_actq_fwd', ad


def _actq_bwd(is_bf16):
    def ad(g, b, v):             # (x, g, dx, K, clip, qmax); grid M
        x, gy, dx, K, clip, qmax = v
        return [x, I(int(is_bf16)), gy, dx, K, clip, qmax, I(g[0])]
    return 'camx_actq_bwd', ad


_CORE = {
    'embedding_f32': _rows('camx_embedding_f32'), 'rmsnorm_f32': _rows('camx_rmsnorm_f32'),
    'silu_mul_bf16': ('camx_silu_mul_bf16', lambda g, b, v: [v[0], v[1], v[2], L64(_val(v[3]))]),
    'residual3': ('camx_residual3', lambda g, b, v: [v[0], v[1], v[2], v[3], L64(_val(v[4]))]),
    'cast_bf16': ('camx_cast_bf16', lambda g, b, v: [v[0], v[1], L64(_val(v[2]))]),
    'copy_cols_bf16': ('camx_copy_cols_bf16', lambda g, b, v: list(v[:7]) + [L64(_val(v[7]))]),
}
_FUSE = {'residual_slices_fwd': ('camx_residual_slices_fwd', lambda g, b, v: list(v[:7]) + [L64(_val(v[7]))]),
         'residual_slices_bwd': ('camx_residual_slices_bwd', lambda g, b, v: list(v[:6]) + [L64(_val(v[6]))])}
_ACTQ = {
    'actq_fwd_f32': _actq(False, False), 'actq_fwd_bf16': _actq(True, False),
    'actq_fwd_codes_f32': _actq(False, True), 'actq_fwd_codes_bf16': _actq(True, True),
    'silu_mul_actq_fwd': _rows('camx_silu_mul_actq_fwd'), 'block_entry_fwd': _rows('camx_block_entry_fwd'),
    'actq_bwd_f32': _actq_bwd(False), 'actq_bwd_bf16': _actq_bwd(True),
    'silu_mul_actq_bwd': _rows('camx_silu_mul_actq_bwd'), 'block_entry_bwd': _rows('camx_block_entry_bwd'),
}
_KV = {'own_kv_q8_append': _rows('camx_own_kv_q8_append')}


def _feed(name, rows_at, width_at, per_unit):
    def ad(g, b, v):             # one thread per output value in the reference: the grid must cover them
        need = _val(v[rows_at]) * _val(v[width_at]) * per_unit
        _expect(g[0] * b[0] >= need, f'{name} covers {g[0] * b[0]} < {need} values')
        return list(v)
    return name, ad


_FEED = {'ple_rows_iq4nl': _feed('camx_ple_rows_iq4nl', 3, 4, 32), 'embd_rows_iq4xs': _feed('camx_embd_rows_iq4xs', 3, 4, 256)}
_GG = {'gg_quantize_q8_1': ('camx_gg_quantize_q8_1', _gg_q8_1), 'gg_silu_mul': _plain('camx_gg_silu_mul')}


def _q3m(yarn, q8):
    d = {'q3p_emb': _rows('camx_q3p_emb'), 'q3p_add_rms16': _rows('camx_q3p_add_rms16'), 'q3p_swiglu': _plain('camx_q3p_swiglu')}
    d['q3p_qk_rope_q8' if q8 else 'q3p_qk_rope'] = _qk_rope(yarn, q8)
    return d


def _glue(K):
    return {'pf_rms_mul': _pf_rms_mul(K),
            'pf_hc_post_rms': ('camx_pf_hc_post_rms', lambda g, b, v: list(v) + [I(K)]),
            'pf_hc_post': _plain('camx_pf_hc_post'), 'pf_hc_mean': _plain('camx_pf_hc_mean'),
            'pf_gdn_conv': ('camx_pf_gdn_conv', lambda g, b, v: list(v) + [I(0)]),
            'pf_conv_state': ('camx_pf_conv_state', lambda g, b, v: list(v) + [I(0)]),
            'pf_add_sum': ('camx_pf_add_sum', lambda g, b, v: [v[0], v[1], v[2], L64(_val(v[3]))]),
            'pf_silu_bf16': _plain('camx_pf_silu_bf16'), 'pf_to_bf16': _plain('camx_pf_to_bf16'),
            'pf_ple_gate': _rows('camx_pf_ple_gate'), 'pf_ple_conv': _plain('camx_pf_ple_conv'), 'pf_ple_hist': _plain('camx_pf_ple_hist')}


def _pf_kv_append16(g, b, v):     # the PREFILL_KV_F16 build of pf_kv_append: (k, ldk, v, ldv, M, cache, pos0, rows, err); grid T
    k, ldk, vv, ldv, M, cache, pos0, rows, err = v
    return [k, ldk, vv, ldv, cache, M, pos0, rows, err, I(g[0])]


_ATTN = {'pf_qk_nr': ('camx_pf_qk_nr', _pf_qk_nr), 'pf_hadamard': _plain('camx_pf_hadamard'), 'pf_kv_append': _rows('camx_pf_kv_append'),
         'pf_gate_mul': _gate(0), 'pf_hc_avg': _plain('camx_pf_hc_avg')}
def _gdn_norm(silu):
    return 'camx_pf_gdn_norm', lambda g, b, v: list(v) + [L64(g[0]), I(silu)]     # one workgroup per (token, value head) in the reference


_GDN = {'pf_gdn_l2': ('camx_pf_gdn_l2', _pf_gdn_l2), 'pf_gdn_gates': _plain('camx_pf_gdn_gates'), 'pf_gdn_norm': _gdn_norm(0)}
_GDN_SILU = dict(_GDN, pf_gdn_norm=_gdn_norm(1))                                   # the code objects built with PF_GDN_SILU (qwen35moe / qwen3next)
_Q35 = {'q35p_add_rms16': _rows('camx_q35p_add_rms16'), 'q35p_gate_mul16': _gate(1),
        'q35p_gdn_norm16': ('camx_q35p_gdn_norm16', lambda g, b, v: list(v) + [L64(g[0])]), 'q35p_kv_append16': _rows('camx_q35p_kv_append16')}

SYMBOLS = {
    'core': _CORE, 'fuse': _FUSE, 'actq': _ACTQ, 'kv_codec': _KV, 'prefill_feed': _FEED, 'k3_gguf': _GG, 'k3_gguf_swiglu': _GG,
    'q3m_prefill': _q3m(False, False), 'q3m_prefill_kvq8': _q3m(False, True), 'q3m_prefill_yarn': _q3m(True, False),
    'q3m_prefill_kvq8_yarn': _q3m(True, True), 'q35_prefill': _Q35,
    'prefill_glue': _glue(2560), 'prefill_glue_q35': _glue(2048), 'prefill_glue_q35d': _glue(5120),
    'prefill_attn': _ATTN, 'prefill_attn_q35': _ATTN, 'prefill_attn_q35d': _ATTN,
    'prefill_attn_f16': dict(_ATTN, pf_kv_append=('camx_q35p_kv_append16', _pf_kv_append16)),      # fp16 cache rows (python/caminus/prefill/attn.py:150-155)
    'prefill_gdn': _GDN, 'prefill_gdn_q35': _GDN_SILU,
    'prefill_mmq_glue': {},      # its quantizers are template instances in the reference: caminus_amd.prefill.mmq binds them
    'camx': {},                  # direct access to every C entry point by its own name (Module('camx').camx_...)
}


class Kernel:
    """one entry point; called like the reference's Kernel: (grid, block, *args, shmem=0, stream=None)"""

    def __init__(self, fn, name, adapter):
        self.fn, self.name, self._adapt = fn, name, adapter

    def lds_bytes(self):
        """static LDS per workgroup is an internal of this library's kernels and not part of the surface"""
        return 0

    def __call__(self, grid, block, *args, shmem=0, stream=None):
        vals = [ctypes.c_void_p(a.data_ptr()) if isinstance(a, torch.Tensor) else a for a in args]
        grid, block = (tuple(int(x) for x in grid) + (1, 1))[:3], (tuple(int(x) for x in block) + (1, 1))[:3]
        s = torch.cuda.current_stream().cuda_stream if stream is None else stream
        r = RECORD
        if r is not None and r.intercept(self, grid, block, vals, shmem, s):
            return
        check(self.fn(*self._adapt(grid, block, vals), ctypes.c_void_p(s)))
        if r is not None:
            r.launched(self, grid, block, vals, shmem, s)


class Module:
    """the kernels of one reference code object, served by libcamx.so on the current device"""

    def __init__(self, name):
        if name not in SYMBOLS:
            raise FileNotFoundError(_kernels.missing_message(name, BUILD, BUILD_FROM) + f' ({name} is not a module of this library)')
        self.handle = hip()                 # FileNotFoundError when libcamx.so is absent
        self._name, self._table, self._fns = name, SYMBOLS[name], {}
        if name not in LOADED:
            LOADED.append(name)

    def __getattr__(self, sym):
        if sym.startswith('_') or sym == 'handle':
            raise AttributeError(sym)
        if sym not in self._fns:
            if sym in self._table:
                cname, adapter = self._table[sym]
            elif self._name == 'camx' and sym.startswith('camx_'):
                cname, adapter = sym, (lambda g, b, v: list(v))
            else:
                raise AttributeError(f'{self._name} has no kernel {sym}')
            self._fns[sym] = Kernel(getattr(self.handle, cname), sym, adapter)
        return self._fns[sym]
