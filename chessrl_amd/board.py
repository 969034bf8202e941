"""Host-side board functions with the reference's names and return types.

fen_to_tensor / encode_fens mirror utils/fen_encoder.py:5-38 and utils/parse.py:71-75;
legal_move_mask mirrors the mask loop of model_bis.py:373-380. All of them run in the
C++ library (no python-chess).
"""
import ctypes as C

import numpy as np

from . import _lib
from ._lib import check, lib, str_array


def fen_to_tensor(fen):
    """FEN -> np.float32[8,8,19], indexed [7-rank, file, plane]."""
    out = np.empty((8, 8, _lib.NUM_PLANES), np.float32)
    check(lib().crl_fen_to_planes(fen.encode(), out.ctypes.data), "crl_fen_to_planes")
    return out


def encode_fens_np(fens, threads=0):
    out = np.empty((len(fens), 8, 8, _lib.NUM_PLANES), np.float32)
    if len(fens):
        check(lib().crl_encode_fens(str_array(fens), len(fens), out.ctypes.data, threads), "crl_encode_fens")
    return out


def encode_fens(fen_array):
    """List of FENs -> torch.float32[B,8,8,19] on the CPU (utils/parse.py:71-75)."""
    import torch
    return torch.from_numpy(encode_fens_np(list(fen_array)))


def encode_fens_compact(fens, threads=0):
    """(uint8[B,64] piece codes in token order, uint8[B,4] flags)."""
    ids = np.empty((len(fens), 64), np.uint8)
    flags = np.empty((len(fens), 4), np.uint8)
    if len(fens):
        check(lib().crl_encode_fens_compact(str_array(fens), len(fens), ids.ctypes.data, flags.ctypes.data, threads),
              "crl_encode_fens_compact")
    return ids, flags


def legal_move_masks(fens, leela=False, threads=0, return_counts=False):
    """uint8[B,1929] (or [B,1858] in the side-to-move frame) legal-move masks."""
    v = _lib.VOCAB_LEELA if leela else _lib.VOCAB_RL
    out = np.empty((len(fens), v), np.uint8)
    counts = np.empty(len(fens), np.int32)
    if len(fens):
        fn = lib().crl_legal_masks_leela if leela else lib().crl_legal_masks
        check(fn(str_array(fens), len(fens), out.ctypes.data, counts.ctypes.data, threads), "crl_legal_masks")
    return (out, counts) if return_counts else out


def legal_move_mask(fen, leela=False):
    return legal_move_masks([fen], leela=leela)[0]


def legal_moves(fen):
    """UCI strings of the legal moves (the library's generation order)."""
    buf = C.create_string_buffer(6 * 256)
    n = check(lib().crl_legal_moves(fen.encode(), buf, 256), "crl_legal_moves")
    raw = buf.raw
    return [raw[i * 6:(i + 1) * 6].split(b"\0")[0].decode() for i in range(n)]


def child_fens(fen):
    """(moves, fens) after every legal move: board.push(m); board.fen() (new_paradigm/value.py:336-340)."""
    fb = C.create_string_buffer(96 * 256)
    mb = C.create_string_buffer(6 * 256)
    n = check(lib().crl_child_fens(fen.encode(), fb, mb, 256), "crl_child_fens")
    mraw, fraw = mb.raw, fb.raw
    moves = [mraw[i * 6:(i + 1) * 6].split(b"\0")[0].decode() for i in range(n)]
    fens = [fraw[i * 96:(i + 1) * 96].split(b"\0")[0].decode() for i in range(n)]
    return moves, fens


def white_to_move(fen):
    return fen.split()[1] == "w" if len(fen.split()) > 1 else True


def perft(fen, depth):
    return int(lib().crl_perft(fen.encode(), depth))


def random_positions(seed, n, max_plies=80, late_fraction=0.0, late_max_pieces=10,
                     planes=True, masks_rl=False, masks_leela=False, fens=False):
    """Seeded uniform-random legal playouts from the start position.

    Returns a dict with the requested arrays: planes float32[n,8,8,19], masks_rl
    uint8[n,1929], masks_leela uint8[n,1858], fens list[str].
    """
    out = {}
    p = np.empty((n, 8, 8, _lib.NUM_PLANES), np.float32) if planes else None
    mr = np.empty((n, _lib.VOCAB_RL), np.uint8) if masks_rl else None
    ml = np.empty((n, _lib.VOCAB_LEELA), np.uint8) if masks_leela else None
    fb = C.create_string_buffer(96 * max(n, 1)) if fens else None
    check(lib().crl_random_positions(
        C.c_uint64(seed), n, max_plies, float(late_fraction), late_max_pieces,
        p.ctypes.data if planes else None, mr.ctypes.data if masks_rl else None,
        ml.ctypes.data if masks_leela else None, C.addressof(fb) if fens else None), "crl_random_positions")
    if planes:
        out["planes"] = p
    if masks_rl:
        out["masks_rl"] = mr
    if masks_leela:
        out["masks_leela"] = ml
    if fens:
        fraw = fb.raw
        out["fens"] = [fraw[i * 96:(i + 1) * 96].split(b"\0")[0].decode() for i in range(n)]
    return out
