"""Prompt lookup (model::LookupIndex): the proposals a request's own tokens make, host code behind the C ABI."""
import ctypes

import numpy as np

from ._native import lib, check

MINIMUM_MATCH, LONGEST_MATCH = 3, 64
AGREEMENT_TOP, AGREEMENT_CANDIDATE, AGREEMENT_ABSENT, AGREEMENT_UNKNOWN = range(4)


class LookupIndex:
    """A request's tokens and, after the latest, the earlier occurrence of their longest suffix (3 to 64 tokens, the most
    recent one): `match()` is (length, end) with length 0 for none; `proposals(n)` the tokens that followed it."""

    def __init__(self, tokens=()):
        self.handle = ctypes.c_void_p()
        check(lib.spo_lookup_index_create(ctypes.byref(self.handle)))
        if len(tokens):
            self.append(tokens)

    def append(self, tokens):
        a = np.ascontiguousarray(tokens, dtype=np.uint32)
        check(lib.spo_lookup_index_append(self.handle, a.ctypes.data, a.size))

    def match(self):
        length, end = ctypes.c_uint32(), ctypes.c_uint32()
        check(lib.spo_lookup_index_match(self.handle, ctypes.byref(length), ctypes.byref(end)))
        return length.value, end.value

    def proposals(self, count):
        out = np.zeros(max(count, 1), dtype=np.uint32)
        n = lib.spo_lookup_index_proposals(self.handle, count, out.ctypes.data)
        return out[:n].copy()

    def close(self):
        if self.handle:
            lib.spo_lookup_index_destroy(self.handle)
            self.handle = None

    def __del__(self):
        self.close()


def agreement(token, depth, candidates, per_position=16):
    """A lookup token's agreement with the draft's candidates [positions][per_position] at its depth."""
    c = np.ascontiguousarray(candidates, dtype=np.uint32).reshape(-1, per_position)
    return lib.spo_lookup_agreement(int(token), depth, c.ctypes.data, c.shape[0], per_position)
