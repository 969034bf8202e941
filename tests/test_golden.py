"""The CPU oracle against output vectors of the reference's own module code (tests/golden/reference_vectors.npz,
written by tests/golden/make_vectors.py; weights and inputs are regenerated here by the same integer hashing)."""
import os
import sys

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import make_vectors as mv  # noqa: E402  (sizes and input recipes only; nothing of the reference is read here)
from fill import det_fill, fill_state_dict, rig_end_variation  # noqa: E402

from oracle import models as om  # noqa: E402

GOLD = np.load(os.path.join(HERE, "golden", "reference_vectors.npz"))


def filled(module, skip=("pe",)):
    sd = module.state_dict()
    arrays = fill_state_dict({k: tuple(v.shape) for k, v in sd.items() if k not in skip})
    module.load_state_dict({k: torch.from_numpy(v) for k, v in arrays.items()}, strict=False)
    return module.eval()


def gpt_oracle():
    c = mv.GPT_CFG
    return filled(om.GPTOracle(c["n_layer"], c["n_head"], c["n_embd"], c["block_size"], c["vocab_size"]))


def gpt_inputs():
    planes = torch.from_numpy(mv.planes_input("gpt.planes", (mv.GPT_B, 8, 8, 19)))
    idx = torch.from_numpy(mv.token_input("gpt.idx", (mv.GPT_B, mv.GPT_T)))
    return planes, idx


def close(got, want, tol=2e-5):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape
    assert np.abs(got - want).max() <= tol * max(1.0, np.abs(want).max()), np.abs(got - want).max()


def test_fill_is_stable():
    # the hashing must never change under the fixture: a few literal values
    v = det_fill("gpt.planes", (4,), 0.0, 1.0)
    assert v.dtype == np.float32 and np.all((v >= 0) & (v < 1)) and len(set(v.tolist())) == 4
    assert det_fill("a", (3, 2), -1, 1).tobytes() == det_fill("a", (6,), -1, 1).tobytes()
    assert det_fill("a", (6,), -1, 1).tobytes() != det_fill("b", (6,), -1, 1).tobytes()


def test_gpt_64_token_forward_matches_reference_vectors():
    planes, idx = gpt_inputs()
    g = gpt_oracle()
    close(g.forward_last(planes)[:, None, :], GOLD["gpt_last"])
    close(g.forward_tokens(planes, idx[:, :0])[0], GOLD["gpt_last"])


def test_gpt_token_forward_and_loss_match_reference_vectors():
    planes, idx = gpt_inputs()
    g = gpt_oracle()
    close(g.forward_tokens(planes, idx)[0], GOLD["gpt_tok_last"])
    logits, loss, _ = g.forward_tokens(planes, idx, compute_loss=True)
    close(logits[:, mv.TOK_ROWS], GOLD["gpt_tok_rows"])
    close(loss, GOLD["gpt_tok_loss"], 1e-5)


def test_gpt_vectors_would_catch_a_swapped_split():
    # the fixture must be sensitive to the mistakes it is there for: q|k|v taken as k|q|v changes the output
    planes, _ = gpt_inputs()
    g = gpt_oracle()
    C = mv.GPT_CFG["n_embd"]
    with torch.no_grad():
        for blk in g.transformer.h:
            w, b = blk.attn.c_attn.weight, blk.attn.c_attn.bias
            w.copy_(torch.cat((w[C:2 * C], w[:C], w[2 * C:])))
            b.copy_(torch.cat((b[C:2 * C], b[:C], b[2 * C:])))
    assert np.abs(g.forward_last(planes)[:, None, :].numpy() - GOLD["gpt_last"]).max() > 1e-3


def test_greedy_generation_with_forced_tokens_matches_reference_vectors():
    """GPT.generate_sequence(T=0) of model_bis.py:213-268: arg-max of the oracle's last-token logits, fed back through
    the oracle's rule bookkeeping, step by step."""
    planes, _ = gpt_inputs()
    g = gpt_oracle()
    arrays = rig_end_variation(fill_state_dict({k: tuple(v.shape) for k, v in g.state_dict().items() if k != "pe"}))
    g.load_state_dict({k: torch.from_numpy(v) for k, v in arrays.items()}, strict=False)
    want = GOLD["gpt_generated"].astype(np.int64)
    steps = want.shape[1] - 1
    assert steps == mv.GPT_CFG["block_size"] - 65
    raw = torch.zeros(mv.GPT_B, 0, dtype=torch.int64)
    seq = om.apply_generation_rules(raw)
    for _ in range(steps):
        nxt = g.forward_tokens(planes, seq)[0][:, 0].argmax(-1, keepdim=True)
        raw = torch.cat((raw, nxt), dim=1)
        seq = om.apply_generation_rules(raw)
    assert seq.tolist() == want.tolist()
    rows = want.tolist()
    assert any(1925 in r and 1927 in r for r in rows) and any(1925 not in r for r in rows)


def test_bt4_forward_matches_reference_vectors():
    c = mv.BT4_CFG
    m = filled(om.BT4Oracle(c["num_layers"], c["d_model"], c["d_ff"], c["num_heads"]))
    planes = torch.from_numpy(mv.planes_input("bt4.planes", (mv.BT4_B, mv.BT4_S, 8, 8, 19)))
    pol, wdl = m.forward_pv(planes.reshape(-1, 8, 8, 19))
    close(pol.reshape(mv.BT4_B, mv.BT4_S, -1), GOLD["bt4_policy"])
    close(wdl.reshape(mv.BT4_B, mv.BT4_S, 3), GOLD["bt4_value"])


def test_relative_attention_matches_reference_vectors():
    """The attention sub-layer alone, with a position table that is not the sinusoid (a swapped u/v offset or a
    shift applied to the wrong term would pass a test whose table is symmetric enough)."""
    c = mv.BT4_CFG
    C, H = c["d_model"], c["num_heads"]
    at = om.BT4Oracle(1, C, c["d_ff"], H).layers[0].attention
    arrays = fill_state_dict({"attention." + k: tuple(v.shape) for k, v in at.state_dict().items()})
    at.load_state_dict({k[len("attention."):]: torch.from_numpy(v) for k, v in arrays.items()})
    x = torch.from_numpy(det_fill("attn.x", (mv.ATTN_B, 64, C), -1.0, 1.0))
    pe = torch.from_numpy(det_fill("attn.pe", (1, 64, C), -1.0, 1.0))[0]
    with torch.no_grad():
        close(om.relative_attention(at, x, pe, H), GOLD["attn_out"])


def test_leela_mirror_table_matches_reference_vectors():
    """mapping_black of Leela/compare_policy.py:469-487, all 1858 entries, against the library's host table."""
    from chessrl_amd import vocab
    w, b = vocab.leela_to_rl_maps()
    assert np.array_equal(b.astype(np.int64), GOLD["leela_mapping_black"].astype(np.int64))
    assert np.array_equal(w, np.arange(1858))
    # map_leela_to_rl on four rows, white first and black first: a scatter through those tables
    pol = det_fill("leela.policies", (4, 1858), 0.0, 1.0)
    for first_white, key in ((True, "leela_to_rl_white_first"), (False, "leela_to_rl_black_first")):
        res = np.zeros((4, 1929), dtype=np.float32)
        for r in range(4):
            res[r, w if (r % 2 == 0) == first_white else b] = pol[r]
        assert np.array_equal(res, GOLD[key])
