"""The position-span checks and KV row geometry the launch wrappers share. Mirrors the corresponding helpers of the
reference's python/caminus/engine/k3.py (ContextBoundsError :413-420, check_span :423-437, kv_pos_bytes :530-532,
kv_rows :535-540), and TapeOps: the tape's row ops (python/caminus/engine/k3.py:854-860, 1002-1008, 1057-1089, 1209-1257) with
their Seg field order, each one launch of the library with the position read from a device word. The persistent tape walker of
that module (one kernel that runs a whole layer, matrix products included) is not part of this library."""
import numpy as np

from ..errors import InvalidKVEncoding, NumericalFailure   # noqa: F401  (re-exported as in the reference module)

YARN_TABLE_FLOATS = 65      # freq[64] | mscale appended to the rotary parameter block in the long-context mode


class ContextBoundsError(IndexError):
    """a position (or a lazy-commit count) outside what the caller's buffers hold; raised on the host before any launch"""


def check_span(i0, n, max_ctx, commit=None, ntok=None, what='pass'):
    """positions i0 .. i0 + n - 1 must lie in [0, max_ctx); a commit count (when given) in [0, ntok]"""
    if isinstance(i0, bool) or not isinstance(i0, (int, np.integer)):
        raise ContextBoundsError(f'k3 {what}: position {i0!r} is not an int')
    i0, n = int(i0), int(n)
    if i0 < 0 or n < 1 or i0 + n > max_ctx:
        raise ContextBoundsError(f'k3 {what}: positions {i0} .. {i0 + n - 1} outside the KV cache [0, {max_ctx}) '
                                 f'(max_ctx {max_ctx}; build the engine with a larger max_ctx)')
    if commit is not None:
        if isinstance(commit, bool) or not isinstance(commit, (int, np.integer)) or not 0 <= int(commit) <= ntok:
            raise ContextBoundsError(f'k3 {what}: commit {commit!r} outside [0, {ntok}] (tokens of the previous pass)')


def kv_pos_bytes(M, q8):
    """bytes of one position's [K | V] row with M values each: Q8 blocks of 34 bytes per 32 values, or fp16"""
    return 2 * (M // 32) * 34 if q8 else 4 * M


def kv_rows(cache, M, q8):
    """positions a cache tensor holds, from its byte size"""
    pb = kv_pos_bytes(M, q8)
    nb = cache.numel() * cache.element_size()
    if q8 and M % 32:
        raise ValueError(f'k3 KV cache: {M} values per position is not a whole number of q8_0 blocks')
    if nb % pb or not 0 < nb // pb < 2 ** 31:
        raise ValueError(f'k3 KV cache: {nb} bytes is not a whole number of {pb}-byte positions')
    return nb // pb


# ---- the hot-path ops of the tape as immediate launches -------------------------------------------------------------------------------
# The reference's K3 object appends a Seg per op and runs the whole tape in one persistent launch (python/caminus/engine/k3.py:393-399).
# The tape walker is not part of this library; TapeOps offers the same methods with the same arguments for the row ops this library
# covers, each launched at once through the C ABI's camx_op_* entry points (dep / team / rows_per_task describe the tape's scheduling
# and are accepted and ignored). The position is the tape's own: an int32 word on the device, so a captured graph of these launches
# advances when the caller increments that word.
OWN_BLOCK = {'Q4_K': 144, 'IQ2_S': 82}
OWN_FMT = {'Q4_K': 4, 'IQ2_S': 7}


class TapeOps:
    def __init__(self, T=1, kv_q8_dense=False, kv_error=None, q35=False):
        """T: tokens per pass; kv_q8_dense: kv_append(q8=True) writes the dense Q8 line's blocks with the codec's refusal rules (the
        reference's K3_Q35_KV_Q8 modules) and needs kv_error, the sticky int32 word"""
        import ctypes
        import torch
        from ..device import lib as _lib
        self.T, self.kv_q8_dense, self.kv_error = int(T), bool(kv_q8_dense), kv_error
        self.q35 = bool(q35)            # the dense line's modules: own_add_rms16 at any row length, one unweighted addend, the fp16 copy rounded once
        if self.kv_q8_dense and kv_error is None: raise ValueError('TapeOps: the dense Q8 KV line needs its error word (kv_error)')
        self._C, self._torch, self._L, self._check = ctypes, torch, _lib.load(), _lib.check
        self.params = None              # the pass parameters of gdn_conv (int32 [4] on the device; [1] = tokens of the previous pass to commit)
        self.n = 0

    def _p(self, t):
        return self._C.c_void_p(None if t is None else t.data_ptr())

    def _go(self, name, *args):
        st = self._C.c_void_p(self._torch.cuda.current_stream().cuda_stream)
        self._check(getattr(self._L, name)(*args, st))
        self.n += 1
        return self.n - 1

    def gg_q8_1(self, x, yq, dep=-1, team=-1, silu_scale=None, mul=None):
        I, F = self._C.c_int, self._C.c_float
        n = x.numel(); assert mul is None or (silu_scale is None and mul.numel() == n)
        work = 2 if mul is not None else 0 if silu_scale is None else 1
        return self._go('camx_op_gg_q8_1', self._p(x), self._p(yq), I(n), I(work), F(0.0 if silu_scale is None else silu_scale), self._p(mul))

    def rms_mul(self, x, w, out, eps, dep=-1, team=-1, q8=None):
        I, F = self._C.c_int, self._C.c_float
        K = x.shape[-1]; R = x.numel() // K; wr = w.numel() // K; assert R % wr == 0 and (q8 is None or K % 32 == 0)
        return self._go('camx_op_rms_mul', self._p(x), self._p(w), self._p(out), self._p(q8), I(R), I(wr), I(K), F(eps))

    def own_add_rms16(self, x, nw, h, h16, eps, d=None, slots=0, w=None, dep=-1, team=-1, tokens=1, h16_stride=None):
        I, F = self._C.c_int, self._C.c_float
        n = x.numel() // tokens; hs = n if h16_stride is None else int(h16_stride)
        if n % 256 or not 256 <= n <= 65536: raise ValueError(f'own_add_rms16: n {n} (a multiple of 256, at most 65536)')
        if self.q35 or n > 2048:                                     # (the dense line's modules: kernels/k3_q35_ops.h:79-130)
            if slots > 1 or w is not None or h is None: raise ValueError(f'own_add_rms16: the dense line takes one unweighted addend or none, and the fp32 copy')
            return self._go('camx_op_q35_add_rms16', self._p(x), self._p(d), I(slots), self._p(nw), F(eps), self._p(h), self._p(h16), I(n), I(hs), I(tokens))
        assert 0 <= slots <= 8 and (slots == 0 or d.numel() >= tokens * slots * n) and (w is None or w.numel() >= tokens * slots)
        return self._go('camx_op_own_add_rms16', self._p(x), self._p(d), self._p(w), I(slots), self._p(nw), F(eps), self._p(h), self._p(h16), I(n), I(hs), I(tokens))

    def own_emb(self, w, fmt, vocab, D, tok, x, dep=-1, team=-1, tokens=1, key=False):
        I = self._C.c_int
        if fmt not in OWN_FMT: raise ValueError(f'own_emb: {fmt} (Q4_K, IQ2_S)')
        rb = D // 256 * OWN_BLOCK[fmt]; assert D % 256 == 0 and w.numel() * w.element_size() >= vocab * rb and x.numel() >= tokens * D
        return self._go('camx_op_own_emb', self._p(w), self._p(tok), self._p(x), I(D), I(rb), I(OWN_FMT[fmt]), I(1 if key else 0), I(vocab), I(tokens))

    def own_swiglu16(self, g, u, y16, rows_per_task=1024, dep=-1, team=-1):
        n = g.numel(); assert u.numel() == n and y16.dtype == self._torch.float16 and y16.numel() >= n
        return self._go('camx_op_own_swiglu16', self._p(g), self._p(u), self._p(y16), self._C.c_int(n))

    def own_f16(self, x, out, rows_per_task=1024, dep=-1, team=-1):
        n = x.numel(); assert x.dtype == self._torch.float32 and out.dtype == self._torch.float16 and out.numel() >= n
        return self._go('camx_op_own_f16', self._p(x), self._p(out), self._C.c_int(n))

    def own_moe_sum(self, d, x, slots=1, w=None, rows_per_task=1024, dep=-1, team=-1):
        n = x.numel(); assert d.numel() >= slots * n and (w is None or w.numel() >= slots) and 1 <= slots <= 64
        return self._go('camx_op_own_moe_sum', self._p(d), self._p(w), self._p(x), self._C.c_int(n), self._C.c_int(slots))

    def shexp_add(self, moe, shexp, gate_logit, out, rows_per_task=1024, dep=-1, team=-1):
        n = out.numel(); assert n % self.T == 0 and gate_logit.numel() >= self.T
        return self._go('camx_op_shexp_add', self._p(moe), self._p(shexp), self._p(gate_logit), self._p(out), self._C.c_int(n), self._C.c_int(self.T))

    def add_sum(self, a, b, y, rows_per_task=1024, dep=-1, team=-1):
        return self._go('camx_op_add_sum', self._p(a), self._p(b), self._p(y), self._C.c_int(y.numel()))

    def gdn_gates(self, alpha, beta, dt, a, out, dep=-1, team=-1):
        H = alpha.numel() // self.T
        return self._go('camx_op_gdn_gates', self._p(alpha), self._p(beta), self._p(dt), self._p(a), self._p(out), self._C.c_int(H), self._C.c_int(self.T))

    def gdn_norm(self, o, w, z, out, H, S, eps, dep=-1, team=-1, q8=None, silu=False):
        """silu: the reference's K3_GDN_SILU modules (silu(z) in place of sigmoid(z))"""
        I, F = self._C.c_int, self._C.c_float
        if q8 is not None: assert S % 32 == 0
        return self._go('camx_op_gdn_norm', self._p(o), self._p(w), self._p(z), self._p(out), self._p(q8), I(self.T * H), I(S), F(eps), I(1 if silu else 0))

    def gdn_norm16(self, o, w, z, out16, H, S, eps, dep=-1, team=-1):
        I, F = self._C.c_int, self._C.c_float
        N = self.T * H
        assert o.numel() >= N * S and w.numel() == S and z.numel() >= N * S and out16.dtype == self._torch.float16 and out16.numel() >= N * S
        return self._go('camx_op_gdn_norm16', self._p(o), self._p(w), self._p(z), self._p(out16), I(N), I(S), F(eps))

    def gate_mul(self, a, gate, head_stride, offset, out, dim, rows_per_task=256, dep=-1, team=-1, q8=None):
        I = self._C.c_int
        n = a.numel()
        if q8 is not None: assert n % 32 == 0 and rows_per_task % 32 == 0
        return self._go('camx_op_gate_mul', self._p(a), self._p(gate), I(head_stride), I(offset), self._p(out), self._p(q8), I(n), I(dim))

    def qk_nr(self, x, head_stride, heads, dim, w, pos, out, n_rot, theta_scale, eps, dep=-1, team=-1):
        I, F = self._C.c_int, self._C.c_float
        eb = int(np.array([eps], dtype=np.float32).view(np.int32)[0])
        return self._go('camx_op_qk_nr', self._p(x), I(head_stride), I(heads), I(dim), self._p(w), self._p(pos), self._p(out), I(n_rot), F(theta_scale), I(eb), I(self.T))

    def kv_append(self, k, v, cache, pos, q8=False, dep=-1, team=-1):
        I = self._C.c_int
        if k.numel() % self.T: raise ValueError('kv_append: K must contain a whole row per pass token')
        M = k.numel() // self.T
        rows = kv_rows(cache, M, q8)
        if rows < self.T: raise ValueError('kv_append: fewer physical cache rows than pass tokens')
        work = (2 if self.kv_q8_dense else 1) if q8 else 0
        err = self.kv_error
        if err is None: raise ValueError('kv_append: an int32 error word (kv_error) receives the span / codec bits')
        return self._go('camx_op_kv_append', self._p(k), self._p(v), self._p(cache), self._p(pos), I(M), I(work), self._p(err), I(rows), I(self.T))

    def hadamard(self, x, n, rows_per_task=1, dep=-1, team=-1):
        assert n in (64, 128, 256) and x.numel() % n == 0
        if (isinstance(rows_per_task, (bool, np.bool_)) or not isinstance(rows_per_task, (int, np.integer))
                or not 1 <= rows_per_task < 2 ** 31 or not 0 < x.numel() // n < 2 ** 31):
            raise ValueError('k3 Q8 Hadamard: positive int32 chunk/task counts required')
        I = self._C.c_int
        return self._go('camx_op_hadamard', self._p(x), I(x.numel() // n), I(n), I(int(rows_per_task)))

    def gate_mul16(self, a, gate, head_stride, offset, out16, dim, rows_per_task=256, dep=-1, team=-1):
        I = self._C.c_int
        n = a.numel(); assert n % dim == 0 and gate.numel() >= (n // dim - 1) * head_stride + offset + dim
        assert out16.dtype == self._torch.float16 and out16.numel() >= n
        return self._go('camx_op_gate_mul16', self._p(a), self._p(gate), I(head_stride), I(offset), self._p(out16), I(n), I(dim))

    def hadamard_gate_mul16(self, a, n, gate, head_stride, offset, out16, dim, keep=True, dep=-1, team=-1):
        """hadamard(a, n) then gate_mul16(a, gate, head_stride, offset, out16, dim) in one launch (the dense Q8 line's attention output:
        python/caminus/engine/q35_dense.py:419-420); keep: a is left transformed, as the in-place op leaves it"""
        I = self._C.c_int
        ne = a.numel(); assert n in (64, 128, 256) and dim % n == 0 and ne % dim == 0
        assert gate.numel() >= (ne // dim - 1) * head_stride + offset + dim and out16.dtype == self._torch.float16 and out16.numel() >= ne
        return self._go('camx_op_hadamard_gate_mul16', self._p(a), self._p(a if keep else None), self._p(gate), I(head_stride), I(offset), self._p(out16),
                        I(ne), I(dim), I(n))

    def gdn_l2(self, x, out, heads, dim, eps, x_stride=0, dep=-1, team=-1):
        I, F = self._C.c_int, self._C.c_float
        return self._go('camx_op_gdn_l2', self._p(x), self._p(out), I(heads), I(dim), F(np.float32(eps / dim)), I(x_stride), I(self.T))

    def gdn_conv(self, x, w, state, out, xprev, rows_per_task=256, dep=-1, team=-1):
        I = self._C.c_int
        C_ = x.numel() // self.T; assert xprev.numel() >= x.numel()
        if self.params is None: raise ValueError('gdn_conv: set TapeOps.params (int32 [4] on the device; [1] = tokens to commit)')
        return self._go('camx_op_gdn_conv', self._p(w), self._p(state), self._p(x), self._p(self.params), self._p(out), self._p(xprev), I(C_), I(self.T))

    # the two chains the reference's dense engine appends back to back (python/caminus/engine/q35_dense.py:399-400, 409-418), one launch each
    def gdn_conv_l2(self, x, w, state, out, xprev, qk, heads, dim, eps, dep=-1, team=-1):
        I, F = self._C.c_int, self._C.c_float
        C_ = x.numel() // self.T
        if dim != 128: raise ValueError('gdn_conv_l2: key heads of 128 values')
        if self.params is None: raise ValueError('gdn_conv_l2: set TapeOps.params (int32 [4] on the device; [1] = tokens to commit)')
        return self._go('camx_op_gdn_conv_l2', self._p(w), self._p(state), self._p(x), self._p(self.params), self._p(out), self._p(xprev), self._p(qk), I(C_), I(self.T),
                        I(heads), F(np.float32(eps / dim)))

    def gdn_conv_l2_gates(self, x, w, state, out, xprev, qk, heads, dim, eps, alpha, beta, dt, a, gates, dep=-1, team=-1):
        """gdn_gates beside gdn_conv -> gdn_l2 in one launch (python/caminus/engine/q35_dense.py:396-400)"""
        I, F = self._C.c_int, self._C.c_float
        C_ = x.numel() // self.T; H = alpha.numel() // self.T
        if dim != 128: raise ValueError('gdn_conv_l2_gates: key heads of 128 values')
        if self.params is None: raise ValueError('gdn_conv_l2_gates: set TapeOps.params (int32 [4] on the device; [1] = tokens to commit)')
        return self._go('camx_op_gdn_conv_l2_gates', self._p(w), self._p(state), self._p(x), self._p(self.params), self._p(out), self._p(xprev), self._p(qk), I(C_),
                        I(self.T), I(heads), F(np.float32(eps / dim)), self._p(alpha), self._p(beta), self._p(dt), self._p(a), self._p(gates), I(H))

    def qk_nr_q8(self, q, q_head_stride, heads, k, v, kv_heads, qn, kn, pos, qo, cache, n_rot, theta_scale, eps, dep=-1, team=-1):
        I, F = self._C.c_int, self._C.c_float
        M = kv_heads * 256
        rows = kv_rows(cache, M, True)
        return self._go('camx_qk_nr_q8', self._p(q), I(q_head_stride), I(heads), self._p(k), I(M), self._p(v), I(M), I(kv_heads), self._p(qn), self._p(kn), I(n_rot),
                        F(theta_scale), F(eps), I(0), self._p(pos), self._p(None), self._p(qo), self._p(cache), I(rows), self._p(self.kv_error), I(self.T))

    def qk_nr_kv(self, q, q_head_stride, heads, k, k_head_stride, v, kv_heads, dim, qn, kn, pos, qo, cache, n_rot, theta_scale, eps, ko=None, q8=False,
                 dep=-1, team=-1):
        """qk_nr(k) -> kv_append(ko, v, cache, pos, q8) and qk_nr(q) in one launch (the fp16 and q8_0 cache lines:
        python/caminus/engine/q3moe_one.py:316-318); ko: the buffer the separate ops pass between them, written only if given"""
        I, F = self._C.c_int, self._C.c_float
        M = kv_heads * dim
        if q8 and self.kv_q8_dense: raise ValueError('qk_nr_kv: the dense Q8 line has its own chain (qk_nr_q8)')
        if v.numel() != self.T * M: raise ValueError('qk_nr_kv: V must contain a whole row per pass token')
        rows = kv_rows(cache, M, q8)
        if rows < self.T: raise ValueError('qk_nr_kv: fewer physical cache rows than pass tokens')
        if self.kv_error is None: raise ValueError('qk_nr_kv: an int32 error word (kv_error) receives the span bit')
        return self._go('camx_qk_nr_kv', self._p(q), I(q_head_stride), I(heads), self._p(qn), self._p(k), I(k_head_stride), self._p(v), I(M), I(kv_heads), self._p(kn),
                        I(dim), I(n_rot), F(theta_scale), F(eps), I(0), self._p(pos), self._p(None), self._p(qo), self._p(ko), self._p(cache), I(1 if q8 else 0),
                        I(rows), self._p(self.kv_error), I(self.T))
