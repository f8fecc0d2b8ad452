"""Host-side buffer checks that run before a launch.

Two rules, both refusals are ValueError and nothing is launched after one:
  1. extent   - a buffer must hold, inside its OWN view, every element the kernel touches through its pointer. Workspaces
                are single allocations carved into views; checking against the end of the storage would let a short view
                spill into its neighbour.
  2. aliasing - a buffer the kernel writes may not share a byte with any other buffer of the launch, except a pair the
                kernel declares as an exact in-place use (same first byte, same length).

The public names, argument meanings and messages follow the reference's python/caminus/device/bufcheck.py:29-106
(`aligned`, `view_bytes`, `span`, `disjoint`, `LaunchCheck`), so its launch wrappers and their tests read the same here.
"""
import torch

ALIGN = 256          # block alignment of workspace layouts


def aligned(layout, a=ALIGN):
    """a {name: bytes} layout with each entry padded to a multiple of `a` bytes"""
    out = {}
    for name, nbytes in layout.items():
        out[name] = ((nbytes + a - 1) // a) * a
    return out


def view_bytes(t):
    """bytes covered by a contiguous tensor's own elements"""
    return t.numel() * t.element_size()


def span(t, nbytes):
    """[first, past-the-last) device byte a kernel touches through t's pointer"""
    first = t.data_ptr()
    return first, first + int(nbytes)


def _refuse_overlaps(op, ranges, writes, same_ok):
    """ranges {name: (lo, hi)} in declaration order; the first clash of each written buffer is the one reported"""
    inplace = [frozenset(pair) for pair in same_ok]

    def describe_allowed():
        if not inplace:
            return ' (this kernel has no in-place form)'
        return ' (exact in-place allowed only for ' + ', '.join('/'.join(sorted(p)) for p in inplace) + ')'

    for w in writes:
        if w not in ranges:
            continue
        wlo, whi = ranges[w]
        for other, (lo, hi) in ranges.items():
            if other == w or whi <= lo or hi <= wlo:
                continue
            identical = (lo, hi) == (wlo, whi)
            if identical and frozenset((w, other)) in inplace:
                continue
            verb = 'is the same buffer as' if identical else 'partially overlaps'
            raise ValueError(f'{op}: {w} [{wlo:#x}, {whi:#x}) {verb} {other} [{lo:#x}, {hi:#x}){describe_allowed()}')


def disjoint(op, bufs, writes, same_ok=()):
    """the aliasing rule on byte counts: bufs {name: (tensor or None, bytes touched)}, writes = names the kernel writes"""
    ranges = {}
    for name, (t, nbytes) in bufs.items():
        if t is not None and int(nbytes) > 0:
            ranges[name] = span(t, nbytes)
    _refuse_overlaps(op, ranges, writes, same_ok)


def _host_mapped(t):
    """whether a CPU tensor is a device-mapped pinned buffer this library accepts in place of a device tensor. The
    reference accepts its own host-mapped KV buffers (python/caminus/device/hip.py:40-64); this library allocates none."""
    return False


class LaunchCheck:
    """Both rules for element-indexed launchers, each buffer stated once.

    check = LaunchCheck(prefix, align=1, short_dtype=False)
    check(dev, op, bufs, writes, same_ok=(), opt=(), names=None)
      bufs   {name: (tensor, dtype, elements[, pointer alignment])}, checked in this order
      opt    names that may be None (an absent optional buffer); any other None is refused
      names  {name: wording} for the per-buffer refusals (the aliasing refusal always uses the keys)
    """
    __slots__ = ('mod', 'align', 'short')

    def __init__(self, mod, align=1, short_dtype=False):
        self.mod = mod
        self.align = int(align)
        self.short = bool(short_dtype)

    def _dtype_name(self, dt):
        return str(dt)[len('torch.'):] if self.short else dt

    def _one(self, dev, label, spec):
        """extent / dtype / alignment of one buffer; returns its touched byte range or None for zero elements"""
        t, dtype, count = spec[0], spec[1], int(spec[2])
        on_device = isinstance(t, torch.Tensor) and (t.device == dev or (t.device.type == 'cpu' and _host_mapped(t)))
        if not on_device or not t.is_contiguous():
            raise ValueError(f'{self.mod}: {label} must be a contiguous tensor on {dev}')
        if t.dtype != dtype:
            raise ValueError(f'{self.mod}: {label} must be {self._dtype_name(dtype)} (is {t.dtype})')
        if t.numel() < count:
            raise ValueError(f'{self.mod}: {label} holds {t.numel()} < {spec[2]} elements (its view; {view_bytes(t)} B)')
        need = spec[3] if len(spec) > 3 else self.align
        first = t.data_ptr()
        if need > 1 and first % need:
            raise ValueError(f'{self.mod}: {label} must be {need}-byte aligned')
        return (first, first + count * t.element_size()) if count > 0 else None

    def __call__(self, dev, op, bufs, writes, same_ok=(), opt=(), names=None):
        ranges = {}
        for name, spec in bufs.items():
            if spec[0] is None and name in opt:
                continue
            r = self._one(dev, names.get(name, name) if names else name, spec)
            if r is not None:
                ranges[name] = r
        _refuse_overlaps(op, ranges, writes, same_ok)
