"""chessrl_amd — MI355X-native batched policy/value forward pass for the ChessRL models.

The compute path is the HIP library behind include/chessrl_amd.h; this package is the
ctypes binding that rebuilds the reference's Python surface (GPT, GPTConfig, BT4,
encode_fens, policy_index, ...) on top of it.
"""
from ._lib import CrlError, LIB_PATH  # noqa: F401
