"""CPU tests: the C++ host substrate against known answers and the pure-Python rules oracle,
and the shape of the C ABI (every declared symbol is exported)."""
import ctypes
import hashlib
import os
import re

import numpy as np
import pytest

from chessrl_amd import _lib, board, models, vocab
from oracle import chess_py

START = "rnbqkbnr/pppppppp/8/8/8/8/PPPPPPPP/RNBQKBNR w KQkq - 0 1"
KIWI = "r3k2r/p1ppqpb1/bn2pnp1/3PN3/1p2P3/2N2Q1p/PPPBBPPP/R3K2R w KQkq -"
POS3 = "8/2p5/3p4/KP5r/1R3p1k/8/4P1P1/8 w - -"
POS4 = "r3k2r/Pppp1ppp/1b3nbN/nP6/BBP1P3/q4N2/Pp1P2PP/R2Q1RK1 w kq - 0 1"
POS5 = "rnbq1k1r/pp1Pbppp/2p5/8/2B5/8/PPP1NnPP/RNBQK2R w KQ - 1 8"
# chessprogramming.org perft results
PERFT = {START: [20, 400, 8902, 197281, 4865609], KIWI: [48, 2039, 97862, 4085603], POS3: [14, 191, 2812, 43238, 674624],
         POS4: [6, 264, 9467, 422333], POS5: [44, 1486, 62379, 2103487]}
REF_FEN = "r1bq1rk1/2pp1ppp/p1n2n2/2b1p3/1pP1P3/1B1P1N2/PP3PPP/RNBQR1K1 b - c3 0 9"  # utils/fen_encoder.py:92


def test_header_symbols_exported():
    hdr = open(os.path.join(os.path.dirname(_lib.LIB_PATH), "..", "include", "chessrl_amd.h")).read()
    declared = set(re.findall(r"\b(crl_[a-z0-9_]+)\s*\(", hdr))
    declared -= {"crl_model_config"}
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    assert b"gfx950" in _lib.lib().crl_version()


def test_vocab_pinned():
    # utils/vocab.py: sizes, hashes, prefix relation, the 66 black promotions and the 5 specials
    assert len(vocab.policy_index) == 1929 and len(vocab.policy_leela) == 1858
    assert hashlib.sha256("\n".join(vocab.policy_leela).encode()).hexdigest() == vocab.POLICY_LEELA_SHA256
    assert hashlib.sha256("\n".join(vocab.policy_index).encode()).hexdigest() == vocab.POLICY_INDEX_SHA256
    assert vocab.policy_index[:1858] == vocab.policy_leela
    assert len(set(vocab.policy_index)) == 1929
    assert vocab.policy_index[1858] == "a2a1q" and vocab.policy_index[1923] == "h2h1b"
    assert vocab.policy_index[1924:] == ["<thinking>", "</thinking>", "end_variation", "end", "padding_token"]
    assert vocab.move_to_index("e2e4") == vocab.policy_index.index("e2e4")
    assert vocab.move_to_index("a7a8n") == vocab.policy_index.index("a7a8")     # model_bis.py:376-377
    assert vocab.move_to_index("a7a8q") == vocab.policy_index.index("a7a8q")
    assert vocab.move_to_index("a1a1") == -1


def test_vocab_against_reference_file_when_present():
    path = "/root/reference/utils/vocab.py"
    if not os.path.exists(path):
        pytest.skip("reference checkout not present")
    import ast
    tree = ast.parse(open(path).read())
    lists = {n.targets[0].id: ast.literal_eval(n.value) for n in tree.body if isinstance(n, ast.Assign)}
    assert lists["policy_index"] == vocab.policy_index
    assert lists["policy_leela"] == vocab.policy_leela


def test_mirror_map_known_answers():
    # Leela/compare_policy.py:526-544: idx 4 (a1f1) stays a1f1 for a white row; idx 5 (a1g1) lands on a8g8 for a black row
    w, b = vocab.leela_to_rl_maps()
    assert vocab.policy_leela[4] == "a1f1" and vocab.policy_index[w[4]] == "a1f1"
    assert vocab.policy_leela[5] == "a1g1" and vocab.policy_index[b[5]] == "a8g8"
    assert np.array_equal(w, np.arange(1858))
    for i in range(1858):  # closed form: rank -> 9 - rank (compare_policy.py:437-463)
        assert vocab.policy_index[b[i]] == chess_py.mirror_uci(vocab.policy_leela[i])
    assert len(set(b.tolist())) == 1858
    assert vocab.policy_index[b[vocab.policy_leela.index("a7a8q")]] == "a2a1q"


@pytest.mark.parametrize("fen", list(PERFT))
def test_perft_cpp(fen):
    for d, n in enumerate(PERFT[fen], start=1):
        assert board.perft(fen, d) == n, (fen, d)


@pytest.mark.parametrize("fen,depth", [(START, 3), (KIWI, 2), (POS3, 3), (POS4, 2), (POS5, 2)])
def test_perft_python_oracle(fen, depth):
    assert chess_py.Position(fen).perft(depth) == PERFT[fen][depth - 1]


def test_fen_to_tensor_hand_written():
    t = board.fen_to_tensor(START)
    assert t.shape == (8, 8, 19) and t.dtype == np.float32
    assert t[:, :, :12].sum() == 32
    assert t[7, 4, 5] == 1 and t[0, 4, 11] == 1            # white king e1 -> row 7, black king e8 -> row 0
    assert t[6, :, 0].sum() == 8 and t[1, :, 6].sum() == 8  # pawns
    assert (t[:, :, 12] == 1).all() and (t[:, :, 14:18] == 1).all()
    assert t[:, :, 13].sum() == 0 and t[:, :, 18].sum() == 0
    # the reference's own sample FEN: black to move, ep square c3 -> token (7-2)*8+2 = 42, no castling
    r = board.fen_to_tensor(REF_FEN)
    assert (r[:, :, 12] == 0).all() and (r[:, :, 14:18] == 0).all()
    assert r[:, :, 13].sum() == 1 and r.reshape(64, 19)[42, 13] == 1
    assert np.allclose(r[:, :, 18], 0.0)
    h = board.fen_to_tensor("8/8/8/4k3/8/8/8/R3K2R w KQ - 150 90")
    assert (h[:, :, 18] == 1.0).all() and (h[:, :, 14] == 1).all() and (h[:, :, 15] == 1).all() and (h[:, :, 16:18] == 0).all()
    h = board.fen_to_tensor("8/8/8/4k3/8/8/8/R3K2R w KQ - 37 90")
    assert np.allclose(h[:, :, 18], 0.37)
    # rights without the rook/king at home are dropped (python-chess clean_castling_rights)
    c = board.fen_to_tensor("4k3/8/8/8/8/8/8/4K2R w KQkq - 0 1")
    assert (c[:, :, 14] == 1).all() and (c[:, :, 15:18] == 0).all()


def test_bad_fen_raises():
    for bad in ["", "8/8/8/8 w - - 0 1", "rnbqkbnr/pppppppp/8/8/8/8/PPPPPPPP/RNBQKBNX w KQkq - 0 1",
                "rnbqkbnr/pppppppp/8/8/8/8/PPPPPPPP/RNBQKBNR x KQkq - 0 1", "rnbqkbnr/pppppppp/8/8/8/8/PPPPPPPP/RNBQKBNR w KQkq e5 0 1"]:
        with pytest.raises(_lib.CrlError):
            board.fen_to_tensor(bad)
    assert board.encode_fens_np([]).shape == (0, 8, 8, 19)
    assert board.legal_move_masks([]).shape == (0, 1929)


def test_planes_and_masks_match_python_oracle():
    r = board.random_positions(7, 160, fens=True, masks_rl=True, masks_leela=True)
    fens = r["fens"] + [START, KIWI, POS3, POS4, POS5, REF_FEN, "8/P7/8/8/8/8/p7/K6k b - - 0 1", "4k3/8/8/8/3Pp3/8/8/4K3 b - d3 0 1"]
    planes = board.encode_fens_np(fens)
    masks, counts = board.legal_move_masks(fens, return_counts=True)
    lmasks = board.legal_move_masks(fens, leela=True)
    ids, flags = board.encode_fens_compact(fens)
    assert np.array_equal(planes[:160], r["planes"]) and np.array_equal(masks[:160], r["masks_rl"]) and np.array_equal(lmasks[:160], r["masks_leela"])
    for i, fen in enumerate(fens):
        assert np.array_equal(planes[i], np.array(chess_py.fen_to_planes(fen), np.float32)), fen
        moves = chess_py.legal_moves_uci(fen)
        assert sorted(moves) == sorted(board.legal_moves(fen)), fen
        assert counts[i] == len(moves)
        assert masks[i].tolist() == chess_py.legal_mask(fen, vocab.policy_index), fen
        assert lmasks[i].tolist() == chess_py.legal_mask_leela(fen, vocab.policy_leela), fen
        # every legal move owns one slot: a knight promotion takes the plain four-character slot,
        # which no other legal move can claim (a pawn reaching the last rank always promotes)
        assert masks[i].sum() == len(moves) and lmasks[i].sum() == len(moves)
        # compact form carries the same information as the planes
        p = planes[i].reshape(64, 19)
        assert np.array_equal(ids[i], np.where(p[:, :12].any(1), p[:, :12].argmax(1) + 1, 0))
        assert flags[i, 0] == p[0, 12] and flags[i, 2] == (p[:, 13].argmax() if p[:, 13].any() else 255)


def test_child_fens_follow_python_chess_conventions():
    moves, fens = board.child_fens(START)
    assert len(moves) == 20
    assert fens[moves.index("e2e4")] == "rnbqkbnr/pppppppp/8/8/4P3/8/PPPP1PPP/RNBQKBNR b KQkq - 0 1"   # ep square only when capturable
    moves, fens = board.child_fens("rnbqkbnr/ppp1pppp/8/8/3pP3/8/PPPP1PPP/RNBQKBNR w KQkq - 0 3".replace("4P3", "4P3"))
    m2, f2 = board.child_fens("rnbqkbnr/ppp1pppp/8/8/3p4/8/PPPPPPPP/RNBQKBNR w KQkq - 0 3")
    assert f2[m2.index("e2e4")].split()[3] == "e3"            # black pawn on d4 can capture en passant
    assert f2[m2.index("a2a4")].split()[3] == "-"
    k, kf = board.child_fens(KIWI + " 0 1")
    assert kf[k.index("e1g1")].split()[0].endswith("R4RK1") and "K" not in kf[k.index("e1g1")].split()[2]


def test_state_dict_tables_match_library():
    for eng, shapes in [
        (models._Engine(_lib.ARCH_GPT64, 3, 256, 8, 1024), models.gpt_shapes(3, 256)),
        (models._Engine(_lib.ARCH_BT4, 2, 512, 8, 736), models.bt4_shapes(2, 512, 736, 8)),
        (models._Engine(_lib.ARCH_BT4CLASS, 2, 1024, 32, 1536), models.bt4_shapes(2, 1024, 1536, 32, True)),
    ]:
        exp = dict(eng.expected_keys())
        for k, n in exp.items():
            need = int(np.prod(shapes[k]))
            assert need == n or (k == "pe" and need >= n), k
        assert set(shapes) - set(exp) <= {"transformer.wte.weight"}
    with pytest.raises(_lib.CrlError):
        models._Engine(_lib.ARCH_GPT64, 2, 250, 8, 1000)      # head dim must be 32 or 64
    # the attention-policy head of BT4 / BT4-class needs d_model in whole 64s; GPT64 (no such head) takes 96
    for arch in (_lib.ARCH_BT4, _lib.ARCH_BT4CLASS):
        with pytest.raises(_lib.CrlError, match="multiple of 64"):
            models._Engine(arch, 2, 96, 3, 256)
    models._Engine(_lib.ARCH_GPT64, 1, 96, 3, 384)
    e = models._Engine(_lib.ARCH_GPT64, 1, 256, 8, 1024)
    with pytest.raises(_lib.CrlError):
        _lib.check(_lib.lib().crl_model_set_weight(e.handle, b"nope", None, 0))
    assert abs(models._Engine(_lib.ARCH_GPT64, 6, 256, 8, 1024).flops_per_position() / 1e9 - 0.618) < 0.002   # 2*MAC formula
    assert abs(models._Engine(_lib.ARCH_BT4CLASS, 15, 1024, 32, 1536).flops_per_position() / 1e9 - 15.9) < 0.1


def test_no_cpu_fallback():
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    m = models.GPT(models.GPTConfig(block_size=256, vocab_size=1929, n_layer=1, n_head=8, n_embd=256))
    with pytest.raises(_lib.CrlError):
        m.forward((torch.zeros(1, 8, 8, 19), None))


def test_gemm_split_rejects_bad_arguments_before_any_launch():
    """crl_gemm_split checks its arguments on the host: a split outside (0, N) or off a multiple of 8, a tile code that has
    no two-output form, null outputs. Each is CRL_ERR_ARG with a message, with or without a GPU (nothing is launched)."""
    L = _lib.lib()
    buf = (ctypes.c_uint8 * 4096)()
    ptr = ctypes.cast(buf, ctypes.c_void_p)

    def call(C=ptr, C2=ptr, nsplit=256, N=288, tile=0, in_dt=_lib.FP8):
        return L.crl_gemm_split(ptr, 64, ptr, 64, C, 256, C2, 32, nsplit, 16, N, 64, in_dt, _lib.BF16, None, 1.0, tile, None)

    for kw in (dict(nsplit=0), dict(nsplit=288), dict(nsplit=300), dict(nsplit=4), dict(tile=2), dict(tile=13), dict(C2=None), dict(C=None),
               dict(in_dt=_lib.F32)):
        assert call(**kw) == -1, kw   # CRL_ERR_ARG
        assert b"crl_gemm_split" in L.crl_last_error()


def test_late_game_positions_match_python_oracle():
    """The rollout-scoring sweep draws 30 % of its positions from playouts continued until at most 10 pieces remain
    (sparser legal masks): planes, both masks and the piece counts against the pure-Python rules."""
    r = board.random_positions(1, 120, late_fraction=0.3, fens=True, masks_rl=True, masks_leela=True)
    late = 0
    for i, fen in enumerate(r["fens"]):
        pieces = sum(ch.isalpha() for ch in fen.split()[0])
        late += pieces <= 10
        assert np.array_equal(r["planes"][i], np.array(chess_py.fen_to_planes(fen), np.float32)), fen
        assert r["masks_rl"][i].tolist() == chess_py.legal_mask(fen, vocab.policy_index), fen
        assert r["masks_leela"][i].tolist() == chess_py.legal_mask_leela(fen, vocab.policy_leela), fen
    assert 20 <= late <= 55, late           # about 30 % of 120
    # the same seed without the late-game share leaves the other positions untouched in kind: none forced to <= 10 pieces
    base = board.random_positions(1, 120, fens=True)["fens"]
    assert sum(sum(ch.isalpha() for ch in f.split()[0]) <= 10 for f in base) < late
    # seeded: the same call gives the same positions
    again = board.random_positions(1, 120, late_fraction=0.3, fens=True)["fens"]
    assert again == r["fens"]


def test_fp8_checkpoint_layout_loads():
    """A checkpoint of the reference's fp8 model (model_fp8.py, trained by pretrain_fp8.py:12-17 with vocab_size 1936):
    lm_head / wte carry 7 padding rows, and transformer_engine's Linear modules add '<module>._extra_state' entries.
    Both load; the first 1929 rows are the moves."""
    import torch
    cfg = models.GPTConfig(block_size=256, vocab_size=1936, n_layer=1, n_head=8, n_embd=256)
    m = models.GPT(cfg, fp8=True)
    sd = m.state_dict()
    assert sd["lm_head.weight"].shape == (1936, 256) and sd["transformer.wte.weight"].shape == (1936, 256)
    g = torch.Generator().manual_seed(0)
    sd["lm_head.weight"] = torch.randn(1936, 256, generator=g) * 0.02
    sd["transformer.wte.weight"] = sd["lm_head.weight"]
    for mod in ("transformer.h.0.attn.c_attn", "transformer.h.0.attn.c_proj", "transformer.h.0.mlp.c_fc", "transformer.h.0.mlp.c_proj", "lm_head"):
        sd[mod + "._extra_state"] = torch.zeros(8, dtype=torch.uint8)
    m.load_state_dict(sd)                                   # strict
    assert torch.equal(m.state_dict()["lm_head.weight"], sd["lm_head.weight"])
    with pytest.raises(RuntimeError):
        m.load_state_dict({**sd, "something.else": torch.zeros(1)})
    with pytest.raises(ValueError):
        models.GPT(models.GPTConfig(block_size=256, vocab_size=1900, n_layer=1, n_head=8, n_embd=256))
    # a 1929-row checkpoint still loads into a 1929-row model, and a padded one into it as well (rows beyond 1929 ignored by the logits)
    m2 = models.GPT(models.GPTConfig(block_size=256, vocab_size=1929, n_layer=1, n_head=8, n_embd=256))
    m2.load_state_dict(sd)
