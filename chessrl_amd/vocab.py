"""Move vocabularies, same names as the reference's utils/vocab.py.

policy_index (1929 entries, utils/vocab.py:9-227) and policy_leela (1858 entries,
utils/vocab.py:229-438) are produced by the library from the generation rule; their
SHA-256 over "\\n".join(list) is pinned below.
"""
import numpy as np

from . import _lib

POLICY_LEELA_SHA256 = "4a901f49851725496e39e34648dd58f240950fa6b72a0bbf6b2816b9af767cc7"
POLICY_INDEX_SHA256 = "4f88911e08f3d3959eb86e060b6f51af4eb3a17fbdd1dd63acfdf2223d36148c"


def _load(fn, n):
    return [fn(i).decode() for i in range(n)]


policy_index = _load(_lib.lib().crl_policy_index, _lib.VOCAB_RL)
policy_leela = _load(_lib.lib().crl_policy_leela, _lib.VOCAB_LEELA)


def move_to_index(uci):
    """policy_index.index(uci) after the trailing-'n' strip of model_bis.py:376-380; -1 if absent."""
    return _lib.lib().crl_move_to_index(uci.encode())


def leela_to_rl_maps():
    """(mapping_white, mapping_black) of Leela/compare_policy.py:470-491 as int32[1858]."""
    w = np.empty(_lib.VOCAB_LEELA, np.int32)
    b = np.empty(_lib.VOCAB_LEELA, np.int32)
    _lib.check(_lib.lib().crl_leela_to_rl_maps(w.ctypes.data, b.ctypes.data), "crl_leela_to_rl_maps")
    return w, b
