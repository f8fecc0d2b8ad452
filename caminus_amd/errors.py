"""Terminal failures shared by the launch wrappers (mirrors python/caminus/errors.py:4-24; no torch import)."""


class NumericalFailure(RuntimeError):
    """numerical state corruption that no reset or retry can repair"""


class InvalidKVEncoding(NumericalFailure):
    """a Q8 KV encoder refused a block: the whole append and the cache state it touched are unusable, even though the
    refused block's own bytes were left alone"""
