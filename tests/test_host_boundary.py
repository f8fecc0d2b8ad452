"""The host side of the boundary, on a machine without a GPU: the C-ABI library loads and exports every declared entry
point, and the launch wrappers validate, refuse and marshal exactly as the reference's do (the style of the reference's
tests/device/test_kv_codec.py: a launch recorder instead of the library, torch.cuda entry points patched to fail, CPU
tensors admitted as if they were device-mapped). No kernel is launched anywhere in this file."""
import contextlib
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from caminus_amd import rope
from caminus_amd.device import bufcheck, kernels, kv_codec as K
from caminus_amd.engine.k3 import ContextBoundsError, check_span, kv_pos_bytes, kv_rows

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---- the library and its header -------------------------------------------------------------------------------------------

def _declared():
    text = re.sub(r'/\*.*?\*/', '', open(os.path.join(ROOT, 'include', 'camx.h')).read(), flags=re.S)
    return sorted(set(re.findall(r'\b(camx_[a-z0-9_]+)\s*\(', text)))


def test_library_exports_every_declared_entry_point():
    path = kernels.library_path()
    if not os.path.isfile(path):
        pytest.skip('libcamx.so is not built in this checkout (python -m caminus_amd.build)')
    lib = ctypes.CDLL(path)
    names = _declared()
    assert len(names) >= 40
    assert [n for n in names if not hasattr(lib, n)] == []
    lib.camx_arch.restype = ctypes.c_char_p
    assert lib.camx_arch() == b'gfx950' and lib.camx_version() >= 1        # host-only calls: no GPU is touched


def test_header_is_plain_c():
    """the header compiles as C11 on its own (no C++ or HIP types in any signature)"""
    import subprocess
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, 't.c')
        open(src, 'w').write('#include "camx.h"\nint (*probe)(void) = camx_version;\nint main(void) { return probe == 0; }\n')
        subprocess.run(['gcc', '-std=c11', '-Wall', '-Werror', '-fsyntax-only', '-I', os.path.join(ROOT, 'include'), src], check=True)


def test_kernel_dir_honours_the_environment(monkeypatch, tmp_path):
    monkeypatch.setenv('CAMINUS_KERNEL_DIR', str(tmp_path))
    d, where = kernels.kernel_dir()
    assert d == str(tmp_path) and 'CAMINUS_KERNEL_DIR' in where
    from caminus_amd.device import lib
    monkeypatch.setattr(lib, '_lib', None)
    with pytest.raises(FileNotFoundError, match='libcamx.so'):           # no fallback: a missing library is loud
        lib.load()


# ---- Q8KVCodec: admission, marshalling, error word ---------------------------------------------------------------------------

class Recorder:
    def __init__(self):
        self.calls = []

    def own_kv_q8_append(self, *args):
        self.calls.append(args)


@pytest.fixture
def codec(monkeypatch):
    def forbidden(*a, **k):
        raise AssertionError('GPU initialization forbidden in this test')
    entered = []
    monkeypatch.setattr(torch.cuda, 'init', forbidden)
    monkeypatch.setattr(torch.cuda, 'device', lambda d: (entered.append(d), contextlib.nullcontext())[1])
    monkeypatch.setattr(torch.cuda, 'synchronize', lambda *a: None)
    monkeypatch.setattr(bufcheck, '_host_mapped', lambda t: True)
    loads = []
    rec = Recorder()
    monkeypatch.setattr(K, 'Module', lambda name: (loads.append(name), rec)[1])
    c = K.Q8KVCodec('cuda:0', module=rec)
    c.rec, c.loads, c.entered = rec, loads, entered
    c.base = dict(k=torch.zeros(160), ldk=96, v=torch.zeros(144), ldv=80, M=64, cache=torch.zeros(4 * 136, dtype=torch.uint8), pos0=1, T=2,
                  err=torch.zeros(1, dtype=torch.int32))
    return c


def _append(c, **changes):
    c.append(**dict(c.base, **changes))


def _refused(c, exc=(ValueError, ContextBoundsError), **changes):
    with pytest.raises(exc):
        _append(c, **changes)
    assert c.rec.calls == [] and c.loads == [] and c.entered == []


def test_codec_needs_an_indexed_gpu():
    K.Q8KVCodec(torch.device('cuda:1'))
    for dev in ('cpu', 'cuda', 0, None):
        with pytest.raises(ValueError):
            K.Q8KVCodec(dev)


def test_codec_marshals_the_reference_argument_order(codec):
    _append(codec)
    (grid, block, k, ldk, v, ldv, M, cache, pos0, rows, err), = codec.rec.calls
    assert grid == (2,) and block == (256,)
    assert k is codec.base['k'] and v is codec.base['v'] and cache is codec.base['cache'] and err is codec.base['err']
    assert [a.value for a in (ldk, ldv, M, pos0, rows)] == [96, 80, 64, 1, 4]
    assert all(isinstance(a, ctypes.c_int) for a in (ldk, ldv, M, pos0, rows))
    assert codec.entered == [torch.device('cuda:0')] and codec.loads == []


def test_codec_loads_the_library_once_and_only_after_validation(codec):
    lazy = K.Q8KVCodec('cuda:0')
    lazy.rec, lazy.loads, lazy.entered, lazy.base = codec.rec, codec.loads, codec.entered, codec.base
    _refused(lazy, k=codec.base['k'][:-1])
    _append(lazy); _append(lazy)
    assert codec.loads == ['kv_codec'] and len(codec.rec.calls) == 2


@pytest.mark.parametrize('change', [
    dict(M=48), dict(M=0), dict(M=True), dict(M=64.0), dict(T=0), dict(T=2 ** 31), dict(ldk=63), dict(ldv=63), dict(pos0=-1),
    dict(rows=0), dict(rows=5),                                          # more rows than the cache view holds
    dict(cache=torch.zeros(4 * 136 + 1, dtype=torch.uint8)),             # not whole rows
    dict(cache=torch.zeros(4 * 136, dtype=torch.int8)),                  # wrong dtype
    dict(cache=np.zeros(4 * 136, np.uint8)),                             # not a tensor
    dict(k=torch.zeros(159)),                                            # last row's M values not inside the view
    dict(v=torch.zeros(143)),
    dict(k=torch.zeros(160, dtype=torch.float64)),
    dict(k=torch.zeros(2, 160)[:, ::2]),                                 # not contiguous
    dict(err=torch.zeros(1, dtype=torch.int64)),
    dict(err=None),
])
def test_codec_refuses_bad_layouts_before_any_launch(codec, change):
    _refused(codec, **change)


def test_codec_span_refusals_are_index_errors(codec):
    _refused(codec, exc=ContextBoundsError, pos0=3)                      # rows 3, 4 of 4
    _refused(codec, exc=ContextBoundsError, pos0=1, rows=2)              # narrowed prefix
    _append(codec, pos0=2)                                               # rows 2, 3: the last legal span
    assert issubclass(ContextBoundsError, IndexError)


def test_codec_refuses_aliasing_of_written_buffers(codec):
    store = torch.zeros(4 * 136 + 64, dtype=torch.uint8)
    cache = store[:4 * 136]
    k_over = store[4 * 136 - 64:].view(torch.float32)                    # last 64 cache bytes + 64 spare = 32 floats
    _refused(codec, k=k_over, ldk=32, M=32, v=torch.zeros(64), ldv=32, cache=cache, T=1)    # 8 rows of 68 bytes
    err_in_cache = store[:4].view(torch.int32)
    _refused(codec, cache=cache, err=err_in_cache)
    shared = torch.zeros(160)
    _append(codec, k=shared, v=shared, ldv=96)                           # K and V may alias each other


def test_codec_check_decodes_the_sticky_word(codec):
    word = torch.zeros(1, dtype=torch.int32)
    codec.check(word)
    for bits, text in ((1, 'span'), (2, 'numerical domain'), (4, 'layout'), (3, 'span, numerical domain'), (8, 'unknown error bits'), (10, 'numerical domain, unknown')):
        word[0] = bits
        with pytest.raises(RuntimeError, match=text):
            codec.check(word)
        assert int(word[0]) == bits                                      # never cleared
    with pytest.raises(ValueError):
        codec.check(torch.zeros(1, dtype=torch.int64))


# ---- shared helpers ---------------------------------------------------------------------------------------------------------

def test_span_and_row_geometry_helpers():
    check_span(0, 4, 4); check_span(np.int64(3), 1, 4)
    for i0, n, cap in ((-1, 1, 4), (0, 0, 4), (2, 3, 4), (4, 1, 4)):
        with pytest.raises(ContextBoundsError):
            check_span(i0, n, cap)
    with pytest.raises(ContextBoundsError):
        check_span(True, 1, 4)
    with pytest.raises(ContextBoundsError):
        check_span(0, 1, 4, commit=5, ntok=4)
    assert kv_pos_bytes(512, True) == 1088 and kv_pos_bytes(512, False) == 2048
    assert kv_rows(torch.zeros(3 * 1088, dtype=torch.uint8), 512, True) == 3
    with pytest.raises(ValueError):
        kv_rows(torch.zeros(3 * 1088 + 1, dtype=torch.uint8), 512, True)


def test_bufcheck_rules():
    a = torch.zeros(64)
    assert bufcheck.aligned({'x': 1, 'y': 256, 'z': 257}) == {'x': 256, 'y': 256, 'z': 512}
    assert bufcheck.view_bytes(a) == 256 and bufcheck.span(a, 16) == (a.data_ptr(), a.data_ptr() + 16)
    bufcheck.disjoint('op', {'in': (a[:32], 128), 'out': (a[32:], 128)}, ('out',))
    with pytest.raises(ValueError, match='partially overlaps'):
        bufcheck.disjoint('op', {'in': (a[:40], 160), 'out': (a[32:], 128)}, ('out',))
    with pytest.raises(ValueError, match='same buffer'):
        bufcheck.disjoint('op', {'in': (a, 256), 'out': (a, 256)}, ('out',))
    bufcheck.disjoint('op', {'in': (a, 256), 'out': (a, 256)}, ('out',), same_ok=(('in', 'out'),))


def test_yarn_mode_surface():
    m = rope.YarnMode(4, 32768)
    assert m.max_ctx == 131072 and m.key() == 'yarn:4:32768:32:1' and m.table(128, 1e6).shape == (65,) and m.table(128, 1e6).dtype == np.float32
    for bad in ((1.0, 32768), (0.5, 32768), (4, 0)):
        with pytest.raises(ValueError):
            rope.YarnMode(*bad)
    with pytest.raises(ValueError):
        rope.yarn_table(64, 1e6, 4, 32768)
    assert rope.mscale(1.0) == 1.0 and rope.mscale(0.5) == 1.0


# ---- the C entry points' own argument checks (host code only: nothing reaches a GPU) -----------------------------------------

P = ctypes.c_void_p(0x7f0000001000)          # a well-aligned address that is never dereferenced
NUL = ctypes.c_void_p(None)
ODD = ctypes.c_void_p(0x7f0000001002)          # two-byte aligned only
ODD1 = ctypes.c_void_p(0x7f0000001001)
Ci, Cf, Cl = ctypes.c_int, ctypes.c_float, ctypes.c_long
ST = ctypes.c_void_p(None)

# name -> (arguments of an empty batch: accepted, returns 0 and launches nothing; [(position, bad value), ...]: each refused with 1)
ENTRY_CASES = {
    'camx_q3p_add_rms16': ([P, P, NUL, Ci(1), P, Cf(1e-6), P, P, Ci(2048), Ci(0)], [(0, NUL), (8, Ci(2047)), (8, Ci(4096)), (3, Ci(9)), (9, Ci(-1)), (7, NUL)]),
    'camx_q35p_add_rms16': ([P, P, P, Cf(1e-6), P, P, Ci(5120), Ci(0)], [(0, NUL), (6, Ci(100)), (7, Ci(-1))]),
    'camx_add_rms_q8_1': ([P, P, NUL, Ci(1), P, Cf(1e-6), P, P, P, Ci(2048), Ci(0)], [(9, Ci(48)), (4, NUL), (3, Ci(-1))]),
    'camx_add_rms_bf16': ([P, P, P, Cf(1e-6), P, P, Ci(5120), Ci(0)], [(0, NUL), (2, NUL), (6, Ci(0)), (7, Ci(-2))]),
    'camx_rmsnorm_f32': ([P, P, P, Ci(896), Cf(1e-6), Ci(0)], [(0, NUL), (2, NUL), (3, Ci(0)), (5, Ci(-1))]),
    'camx_gg_quantize_q8_1': ([P, P, Cl(0), Ci(0), Cf(0), NUL], [(0, NUL), (1, NUL), (3, Ci(3)), (3, Ci(2)), (1, ODD), (2, Cl(-1))]),
    'camx_op_own_emb': ([P, P, P, Ci(2048), Ci(1152), Ci(4), Ci(0), Ci(1000), Ci(0)], [(0, NUL), (2, NUL), (5, Ci(9)), (6, Ci(2)), (3, Ci(100)), (4, Ci(100)), (7, Ci(0))]),
    'camx_q3p_swiglu': ([P, P, P, Ci(0)], [(0, NUL), (2, NUL), (3, Ci(-1))]),
    'camx_silu_mul_bf16': ([P, P, Ci(17408), Cl(0)], [(0, NUL), (2, Ci(0)), (3, Cl(5))]),
    'camx_q3p_qk_rope': ([P, Ci(5120), Ci(32), Ci(4), P, Ci(0), P, P, Ci(0), Ci(0)], [(0, NUL), (4, NUL), (1, Ci(100)), (8, Ci(-1))]),
    'camx_q3p_qk_rope_q8': ([P, Ci(5120), Ci(32), Ci(4), P, Ci(0), P, P, P, Ci(0), Ci(0)], [(8, NUL), (0, NUL)]),
    'camx_pf_qk_nr': ([P, Ci(512), Ci(24), P, Ci(256), Ci(64), Cf(0.5), Cf(1e-6), Ci(0), P, Ci(0), Ci(1)], [(4, Ci(513)), (5, Ci(63)), (5, Ci(258)), (1, Ci(128)), (11, Ci(2))]),
    'camx_q3p_emb': ([P, Ci(1152), Ci(1000), P, P, Ci(2048), Ci(0)], [(0, NUL), (1, Ci(1000)), (5, Ci(2000)), (2, Ci(0))]),
    'camx_emb_gather': ([P, Cl(1152), Ci(1000), P, P, P, Ci(2048), Ci(0), Ci(0)], [(8, Ci(4)), (8, Ci(-1)), (0, NUL), (1, Cl(1151))]),
    'camx_embd_rows_iq4xs': ([P, P, Ci(1000), Ci(0), Ci(8), P, P], [(4, Ci(0)), (4, Ci(33)), (6, NUL), (5, NUL)]),
    'camx_ple_rows_iq4nl': ([P, P, Ci(4), Ci(0), Ci(5), P, P], [(0, ODD1), (2, Ci(0)), (4, Ci(0)), (6, NUL)]),
    'camx_hadamard128': ([P, P, Cl(0)], [(0, NUL), (2, Cl(-1))]),
    'camx_gate_mul': ([P, P, P, Cl(0), Ci(256), Ci(512), Ci(256), Ci(2)], [(7, Ci(3)), (6, Ci(257)), (4, Ci(0))]),
    'camx_residual3': ([P, P, P, P, Cl(0)], [(0, NUL), (4, Cl(-1))]),
    'camx_cast_bf16': ([P, P, Cl(0)], [(1, NUL), (2, Cl(-1))]),
    'camx_actq_fwd': ([P, Ci(1), P, P, P, Ci(2048), Cf(1.0), Ci(7), Ci(0)], [(5, Ci(100)), (5, Ci(8320)), (7, Ci(0)), (0, NUL), (8, Ci(-1))]),
    'camx_actq_bwd': ([P, Ci(1), P, P, Ci(2048), Cf(1.0), Ci(7), Ci(0)], [(2, NUL), (3, NUL), (4, Ci(64))]),
    'camx_silu_mul_actq_bwd': ([P, Ci(4096), Ci(2048), P, P, Cf(1.0), Ci(7), Ci(0)], [(1, Ci(4095)), (1, Ci(4000)), (4, NUL)]),
    'camx_block_entry_bwd': ([P, P, P, P, Ci(14), P, P, P, Ci(896), Cf(1.0), Ci(7), Ci(0)], [(8, Ci(2048)), (4, Ci(13)), (4, Ci(18)), (6, NUL)]),
    'camx_pf_hc_mean': ([P, P, P, P, P, Ci(0), Ci(4), Ci(2560), Cf(0.25)], [(1, NUL), (6, Ci(0)), (3, NUL)]),
}


def test_entry_points_accept_empty_batches_and_refuse_bad_arguments():
    path = kernels.library_path()
    if not os.path.isfile(path):
        pytest.skip('libcamx.so is not built in this checkout (python -m caminus_amd.build)')
    lib = ctypes.CDLL(path)
    for name, case in ENTRY_CASES.items():
        good, bad = case
        fn = getattr(lib, name)
        assert fn(*good, ST) == 0, name
        for pos, val in bad:
            args = list(good); args[pos] = val
            assert fn(*args, ST) == 1, (name, pos)
