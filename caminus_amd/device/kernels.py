"""Where libcamx.so (the gfx950 build of the fused row kernels) is found.

Mirrors the lookup order of the reference's code-object directory (python/caminus/device/kernels.py:64-83): the
CAMINUS_KERNEL_DIR environment variable first, else the package's own directory (an in-tree build). There is no fallback
implementation: a missing library is a FileNotFoundError naming how to build it.
"""
import os

ARCH = 'gfx950'
LIBNAME = 'libcamx.so'
PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))      # the caminus_amd package directory

# reference code-object names whose kernels this library provides (Module(name) accepts exactly these)
PROVIDED = ('core', 'fuse', 'actq', 'kv_codec', 'k3_gguf', 'k3_gguf_swiglu', 'q3m_prefill', 'q3m_prefill_kvq8', 'q3m_prefill_yarn',
            'q3m_prefill_kvq8_yarn', 'q35_prefill', 'prefill_glue', 'prefill_glue_q35', 'prefill_glue_q35d', 'prefill_attn',
            'prefill_attn_q35', 'prefill_attn_q35d', 'prefill_gdn', 'prefill_gdn_q35', 'prefill_mmq_glue', 'camx')


def kernel_dir():
    """(directory, where): where is 'env CAMINUS_KERNEL_DIR' or 'package'"""
    v = os.environ.get('CAMINUS_KERNEL_DIR')
    if v:
        return os.path.abspath(v), 'env CAMINUS_KERNEL_DIR'
    return PKG, 'package'


def library_path():
    d, _ = kernel_dir()
    return os.path.join(d, LIBNAME)


def missing_message(name, d, where):
    hint = ('build it in the checkout with `python -m caminus_amd.build`' if where == 'package'
            else f'the directory comes from {where}')
    return f'{LIBNAME} (kernels of {name}) not found in {d} ({hint})'
