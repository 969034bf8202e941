"""Whole-model parity: the HIP forward (through the C ABI) against the CPU fp32 oracle on the same
seeded positions and weights. Tolerances: WDL max-abs <= 1e-2 and top-1 move agreement >= 99.5 %
(the benchmark's bf16 bar); logits are also compared as a relative RMS error."""
import numpy as np
import pytest
import torch

from chessrl_amd import board, models
from chessrl_amd.vocab import policy_leela
from oracle import models as om

pytestmark = pytest.mark.gpu


def positions(n, seed=1, leela=False):
    r = board.random_positions(seed, n, masks_rl=not leela, masks_leela=leela)
    return torch.from_numpy(r["planes"]), torch.from_numpy(r["masks_leela" if leela else "masks_rl"])


def rel_rms(a, b):
    return ((a - b).pow(2).mean().sqrt() / b.pow(2).mean().sqrt()).item()


def top1_agreement(logits, ref, mask):
    m = (1.0 - mask.float()) * -999.0
    return ((logits + m).argmax(-1) == (ref + m).argmax(-1)).float().mean().item()


def report(name, pol, rpol, mask, wdl=None, rwdl=None):
    msg = "%s: policy rel-rms %.2e, top1 %.4f" % (name, rel_rms(pol, rpol), top1_agreement(pol, rpol, mask))
    if wdl is not None:
        msg += ", wdl max-abs %.2e (prob %.2e)" % ((wdl - rwdl).abs().max().item(), (wdl.softmax(-1) - rwdl.softmax(-1)).abs().max().item())
    print(msg)


def test_gpt_plumbing_config(cuda):
    """The small plumbing configuration: 6 layers, d=256, 8 heads, FFN 1024 GELU, B=256."""
    oracle = om.test_init_(om.GPTOracle(6, 8, 256), seed=0)
    planes, mask = positions(256)
    ref = oracle.forward_last(planes)
    m = models.GPT(models.GPTConfig(block_size=256, vocab_size=1929, n_layer=6, n_head=8, n_embd=256))
    m.load_state_dict(oracle.state_dict())
    logits, loss, targets = m.forward((planes.to(cuda), torch.zeros(256, 0, dtype=torch.long, device=cuda)))
    assert logits.shape == (256, 1, 1929) and loss is None
    pol = logits[:, 0].cpu()
    report("gpt cfg1", pol, ref, mask)
    assert rel_rms(pol, ref) < 1e-2
    assert top1_agreement(pol, ref, mask) >= 0.995
    # batch invariance: a single position equals its row in the batch, any order
    one, _, _ = m.forward((planes[17:18].to(cuda), None))
    assert torch.equal(one[0, 0].cpu(), pol[17])
    perm = torch.randperm(256, generator=torch.Generator().manual_seed(0))
    shuf, _, _ = m.forward((planes[perm].to(cuda), None))
    assert torch.equal(shuf[:, 0].cpu(), pol[perm])


def test_gpt_state_dict_roundtrip_and_move(cuda):
    m = models.GPT(models.GPTConfig(block_size=256, vocab_size=1929, n_layer=2, n_head=8, n_embd=256))
    sd = m.state_dict()
    assert sd["transformer.wte.weight"].shape == (1929, 256) and sd["pe"].shape == (256, 256)
    assert torch.equal(sd["transformer.wte.weight"], sd["lm_head.weight"])
    fen = "r1bq1rk1/2pp1ppp/p1n2n2/2b1p3/1pP1P3/1B1P1N2/PP3PPP/RNBQR1K1 b - c3 0 9"
    legal = set(board.legal_moves(fen))
    legal = {mv[:-1] if mv.endswith("n") else mv for mv in legal}
    for T in (0, 1):
        mv, probs = m.get_move_from_fen_no_thinking(fen, T=T, return_probs=True)
        assert mv in legal
        assert abs(probs.sum().item() - 1) < 1e-4
        if T > 0:
            assert torch.equal((probs > 0).cpu(), torch.from_numpy(board.legal_move_mask(fen)).bool())


@pytest.mark.parametrize("cfg", [(2, 256, 368, 4), (10, 512, 736, 8)])
def test_bt4_torch(cuda, cfg, act="bf16"):
    L, Cm, Fm, H = cfg
    oracle = om.test_init_(om.BT4Oracle(L, Cm, Fm, H), seed=1)
    planes, mask = positions(96, seed=2)
    rpol, rwdl = oracle.forward_pv(planes)
    m = models.BT4(L, Cm, Fm, H, act_dtype=act)
    m.load_state_dict(oracle.state_dict())
    pol = m.forward([planes.view(12, 8, 8, 8, 19).to(cuda)])
    assert pol.shape == (12, 8, 1929)
    pol = pol.view(96, 1929).cpu()
    _, wdl = m.evaluate(planes.to(cuda))
    wdl = wdl.cpu()
    report("bt4 %s %s" % (cfg, act), pol, rpol, mask, wdl, rwdl)
    assert rel_rms(pol, rpol) < (2e-2 if act == "bf16" else 4e-3)
    assert (wdl - rwdl).abs().max() <= (1e-2 if act == "bf16" else 2e-3)
    assert top1_agreement(pol, rpol, mask) >= 0.98


def test_bt4_f16(cuda):
    """The reference trains and runs this model under fp16 autocast (new_paradigm/train_value.py:38)."""
    test_bt4_torch(cuda, (10, 512, 736, 8), "f16")


def test_bt4_value_search(cuda):
    m = models.BT4(2, 256, 368, 4)
    fen = "r3k2r/p1ppqpb1/bn2pnp1/3PN3/1p2P3/2N2Q1p/PPPBBPPP/R3K2R w KQkq - 0 1"
    moves, vals = m.calculate_move_values(fen)
    assert len(moves) == 48 and vals.shape == (48,)
    p = m.get_batch_position_values(board.child_fens(fen)[1])
    assert torch.allclose(p.sum(-1), torch.ones(48, device=cuda), atol=1e-5)
    assert torch.allclose(vals, 0.5 * p[:, 1] + p[:, 2])
    best, probs = m.get_best_move_value(fen, T=0, return_probs=True)
    assert best == moves[int(vals.argmax())] and probs.sum() == 1.0
    assert m.get_best_move_value(fen, T=1) in moves
    assert m.get_move_from_fen_no_thinking(fen, T=1) in {mv[:-1] if mv.endswith("n") else mv for mv in moves}


@pytest.mark.parametrize("cfg", [(2, 256, 384, 8), (4, 1024, 1536, 32)])
@pytest.mark.parametrize("act", ["bf16", "f16"])
def test_bt4class_16bit(cuda, cfg, act):
    L, Cm, Fm, H = cfg
    oracle = om.test_init_(om.BT4ClassOracle(policy_leela, L, Cm, Fm, H), seed=2)
    planes, mask = positions(64, seed=3, leela=True)
    rpol, rwdl = oracle.forward_pv(planes)
    m = models.BT4Class(L, Cm, Fm, H, act_dtype=act)
    m.load_state_dict(oracle.state_dict())
    pol, wdl = m(planes.to(cuda))
    pol, wdl = pol.cpu(), wdl.cpu()
    report("bt4class %s %s" % (cfg, act), pol, rpol, mask, wdl, rwdl)
    # 8 (bf16) or 11 (f16) significant bits per stored activation
    assert rel_rms(pol, rpol) < (2e-2 if act == "bf16" else 4e-3)
    assert (wdl - rwdl).abs().max() <= (1e-2 if act == "bf16" else 2e-3)
    assert top1_agreement(pol, rpol, mask) >= 0.98


@pytest.mark.parametrize("fp8", [False, True])
def test_bt4class_batch_invariance(cuda, fp8):
    """A position's policy and WDL are bit-equal whatever batch it travels in: alone, in 64, in 700 (two GEMM tile
    regimes, and the narrow long-K layers of the value head and the bias generator, whose K slices are a function of
    the layer alone), and in any order."""
    m = models.BT4Class(3, 512, 768, 16, fp8=fp8)
    planes, _ = positions(700, seed=12, leela=True)
    x = planes.to(cuda)
    if fp8:
        m.calibrate(x[:128])
    pol, wdl = m(x)
    # 1, 3, 64, 129, 161, 257 and 320 positions: the 64x64, 128x128 and 256x256 tiles of the trunk products, each with
    # and without a ragged last tile (the e4m3 path re-normalises its residual in all three)
    for sl in (slice(5, 6), slice(0, 3), slice(0, 64), slice(7, 136), slice(0, 161), slice(100, 357), slice(10, 330)):
        p2, w2 = m(x[sl].contiguous())
        assert torch.equal(p2, pol[sl]) and torch.equal(w2, wdl[sl])
    perm = torch.randperm(700, generator=torch.Generator().manual_seed(1))
    p3, w3 = m(x[perm.to(cuda)].contiguous())
    assert torch.equal(p3.cpu(), pol.cpu()[perm]) and torch.equal(w3.cpu(), wdl.cpu()[perm])


@pytest.mark.parametrize("act", ["bf16", "f16"])
def test_bt4class_full_size(cuda, act):
    """The benchmark model at its real size (15 layers, d=1024, 32 heads, FFN 1536) and its benchmark
    initialisation (normal(0, 0.02), zero biases), 256 positions.

    WDL meets the 1e-2 bar in both element types. The top-1 bar (99.5 %) cannot be met by any 16-bit
    pipeline on THIS initialisation: the reference's top-1/top-2 logit gap has a median near 1e-3 while
    the logits' standard deviation is 0.07, so rounding noise of 8 (bf16) or 11 (f16) significant bits
    per stored activation is larger than most gaps. What the test pins instead: the logit error itself,
    and that every position whose reference gap exceeds twice the largest logit error picks the same move."""
    L, Cm, Fm, H = 15, 1024, 1536, 32
    oracle = om.spec_init_(om.BT4ClassOracle(policy_leela, L, Cm, Fm, H), seed=0)
    planes, mask = positions(256, seed=1, leela=True)
    rpol, rwdl = oracle.forward_pv(planes)
    m = models.BT4Class(L, Cm, Fm, H, act_dtype=act)
    m.load_state_dict(oracle.state_dict())
    pol, wdl = m(planes.to(cuda))
    pol, wdl = pol.cpu(), wdl.cpu()
    report("bt4class full size %s" % act, pol, rpol, mask, wdl, rwdl)
    neg = (1.0 - mask.float()) * -999.0
    top2 = (rpol + neg).topk(2, -1).values
    gap = top2[:, 0] - top2[:, 1]
    err = (pol - rpol).abs().max().item()
    same = (pol + neg).argmax(-1) == (rpol + neg).argmax(-1)
    decisive = gap > 2 * err
    print("   logit std %.3e, median gap %.3e, max logit error %.3e, decisive positions %d of %d, agreement on them %.4f, overall %.4f"
          % (rpol.std().item(), gap.median().item(), err, int(decisive.sum()), len(gap),
             same[decisive].float().mean().item() if decisive.any() else 1.0, same.float().mean().item()))
    assert rel_rms(pol, rpol) < (4e-2 if act == "bf16" else 6e-3)
    assert (wdl - rwdl).abs().max() <= (1e-2 if act == "bf16" else 2e-3)
    assert bool(same[decisive].all())
    assert same.float().mean() >= (0.6 if act == "bf16" else 0.9)


def test_bt4class_fp8_vs_emulation(cuda):
    """fp8 path against the quantise->dequantise oracle using the SAME static scales."""
    L, Cm, Fm, H = 3, 512, 768, 16
    oracle = om.test_init_(om.BT4ClassOracle(policy_leela, L, Cm, Fm, H), seed=4)
    calib, _ = positions(64, seed=2, leela=True)
    planes, mask = positions(64, seed=3, leela=True)
    plan = om.Fp8Plan(L)
    plan.recording = True
    oracle.forward_pv(calib, plan)
    plan.recording = False
    rpol, rwdl = oracle.forward_pv(planes, plan)
    bpol, bwdl = oracle.forward_pv(planes)
    m = models.BT4Class(L, Cm, Fm, H, fp8=True)
    m.load_state_dict(oracle.state_dict())
    m.calibrate(calib.to(cuda))
    own = m._engine.get_amax()
    print("amax rel diff (own bf16 calibration vs oracle fp32):", np.abs(own / plan.amax.numpy() - 1).max())
    assert np.abs(own / plan.amax.numpy() - 1).max() < 0.05
    m._engine.set_amax(plan.amax.numpy())
    pol, wdl = m(planes.to(cuda))
    pol, wdl = pol.cpu(), wdl.cpu()
    report("bt4class fp8 vs fp8-emulation", pol, rpol, mask, wdl, rwdl)
    report("bt4class fp8 vs fp32", pol, bpol, mask, wdl, bwdl)
    report("fp8-emulation vs fp32 (oracle only)", rpol, bpol, mask, rwdl, bwdl)
    assert rel_rms(pol, rpol) < 5e-2
    assert (wdl - rwdl).abs().max() <= 2e-2


def test_compact_input_equals_planes(cuda):
    r = board.random_positions(5, 32, fens=True)
    ids, flags = board.encode_fens_compact(r["fens"])
    m = models.BT4Class(2, 256, 384, 8)
    p1, w1 = m(torch.from_numpy(r["planes"]).to(cuda))
    p2, w2 = m._engine.forward_compact(torch.from_numpy(ids).to(cuda), torch.from_numpy(flags).to(cuda))
    assert torch.equal(w1, w2), (w1 - w2).abs().max()
    assert torch.equal(p1, p2), (p1 - p2).abs().max()


def test_graphed_evaluator_replays_match_eager(cuda):
    """A captured forward + masked softmax must reproduce the eager result on every replay, with
    eager work and synchronisations in between."""
    m = models.BT4Class(2, 256, 384, 8)
    ge = m.graphed_evaluator(16, T=1.0)
    for seed in (11, 12, 13, 14):
        r = board.random_positions(seed, 16, masks_leela=True)
        planes, mask = torch.from_numpy(r["planes"]).to(cuda), torch.from_numpy(r["masks_leela"]).to(cuda)
        probs, wdl, am = ge(planes, mask)
        probs, wdl, am = probs.clone(), wdl.clone(), am.clone()
        torch.cuda.synchronize()
        eprobs, ewdl = m.evaluate(planes, legal_mask=mask, T=1.0, want_probs=True)
        torch.cuda.synchronize()
        assert torch.equal(probs, eprobs) and torch.equal(wdl, ewdl)
        assert torch.equal(am.long(), eprobs.argmax(-1))


@pytest.mark.parametrize("arch", ["bt4class", "bt4", "gpt"])
def test_evaluate_fens_pipeline_equals_direct(cuda, arch):
    """The chunked FEN front-end (host encode + upload overlapped with device work) returns exactly what the
    direct path returns for planes and masks built one call at a time."""
    n = 300
    leela = arch == "bt4class"
    r = board.random_positions(11, n, masks_rl=not leela, masks_leela=leela, fens=True)
    fens = r["fens"]
    planes = torch.from_numpy(r["planes"]).to(cuda)
    mask = torch.from_numpy(r["masks_leela" if leela else "masks_rl"]).to(cuda)
    if arch == "bt4class":
        m = models.BT4Class(2, 256, 384, 8)
    elif arch == "bt4":
        m = models.BT4(2, 256, 368, 4)
    else:
        m = models.GPT(models.GPTConfig(block_size=256, vocab_size=1929, n_layer=2, n_head=8, n_embd=256))
    pol, wdl = m._engine.forward(planes)
    ref_probs, ref_best = models.masked_softmax(pol, mask, 1.0, want_probs=True)
    for chunk in (64, 128, 1000):     # ragged last chunk, several chunks in flight, one chunk
        probs, w, best = m.evaluate_fens(fens, T=1.0, chunk=chunk)
        assert torch.equal(probs, ref_probs.cpu())
        assert torch.equal(best, ref_best.cpu().to(torch.int32))
        if arch == "gpt":
            assert w is None
        else:
            assert torch.equal(w, wdl.cpu())
    # arg-max only, temperature 0, and the error path leaves the model usable
    _, _, best0 = m.evaluate_fens(fens[:10], T=0.0, chunk=4, want_probs=False, want_wdl=False)
    assert torch.equal(best0, ref_best.cpu().to(torch.int32)[:10])
    from chessrl_amd._lib import CrlError
    with pytest.raises(CrlError):
        m.evaluate_fens(fens[:5] + ["not a fen"] + fens[5:9], chunk=4)
    probs, _, _ = m.evaluate_fens(fens[:7], chunk=4)
    assert torch.equal(probs, ref_probs.cpu()[:7])
    assert m.evaluate_fens([], chunk=4)[2].numel() == 0


def test_search_1ply_batched(cuda):
    """crl_model_search_1ply (calculate_move_values / get_best_move_value of new_paradigm/value.py:319-400 for many
    roots at once): the same moves, values and arg-max move as the per-position path; values against the fp32 oracle
    evaluated on the child positions; roots without legal moves; reproducible draws; the capacity check."""
    oracle = om.test_init_(om.BT4Oracle(2, 256, 368, 4), seed=3)
    m = models.BT4(2, 256, 368, 4)
    m.load_state_dict(oracle.state_dict())
    fens = list(board.random_positions(21, 40, fens=True)["fens"])
    fens += ["7k/P7/8/8/8/8/8/K7 w - - 0 1",                      # promotions among the children
             "R6k/6pp/8/8/8/8/8/K7 b - - 0 1",                    # checkmated: no legal move
             "7k/5Q2/6K1/8/8/8/8/8 b - - 0 1",                    # stalemate: no legal move
             "r1bq1rk1/2pp1ppp/p1n2n2/2b1p3/1pP1P3/1B1P1N2/PP3PPP/RNBQR1K1 b - c3 0 9"]
    best, per_root = m.get_best_moves_value(fens, T=0, return_values=True)
    assert len(best) == len(fens) and len(per_root) == len(fens)
    worst = 0.0
    for fen, bm, (moves, vals) in zip(fens, best, per_root):
        ref_moves, ref_vals = m.calculate_move_values(fen)
        assert moves == list(ref_moves)
        if not moves:
            assert bm == "" and vals.numel() == 0
            continue
        assert torch.allclose(vals, ref_vals.cpu(), rtol=0, atol=2e-6)
        assert bm == moves[int(torch.argmax(vals))]
        # the oracle on the same children (value.py:343-352)
        _, child = board.child_fens(fen)
        _, wdl = oracle.forward_pv(board.encode_fens(child))
        pr = wdl.softmax(-1)
        want = 0.5 * pr[:, 1] + (pr[:, 2] if board.white_to_move(fen) else pr[:, 0])
        worst = max(worst, (vals - want).abs().max().item())
    print("1-ply search: largest |value - oracle| %.2e" % worst)
    assert worst < 1e-2
    assert best[-3] == "" and best[-2] == ""
    # one call without the value arrays, chunked so that several chunks are in flight
    assert m._engine.search_1ply(fens, T=0.0, chunk=64) == best
    # draws: legal, reproducible, seed-dependent
    d1 = m.get_best_moves_value(fens, T=1.0, seed=5)
    d2 = m.get_best_moves_value(fens, T=1.0, seed=5)
    d3 = m.get_best_moves_value(fens, T=1.0, seed=6)
    assert d1 == d2 and d1 != d3
    for mv, (moves, _) in zip(d1, per_root):
        assert (mv in moves) if moves else mv == ""
    # too little room for the per-child arrays is an error, not an overflow
    import ctypes as C
    from chessrl_amd import _lib
    arr = _lib.str_array(fens[:3])
    vals = torch.empty(4)
    assert _lib.lib().crl_model_search_1ply(m._engine.handle, arr, 3, 64, 0.0, 0, None, None, None, C.c_void_p(vals.data_ptr()), 4, 0) < 0
    gpt = models.GPT(models.GPTConfig(block_size=256, vocab_size=1929, n_layer=1, n_head=8, n_embd=256))
    with pytest.raises(_lib.CrlError):
        gpt.get_best_moves_value(fens[:2])


@pytest.mark.parametrize("t", [1, 37, 192])
def test_gpt_forward_with_move_tokens(cuda, t):
    """GPT.forward((planes, idx), compute_loss) of model_bis.py:171-199: 64 board tokens followed by t move tokens,
    causal attention over all of them; last-token logits, per-token logits and the cross-entropy."""
    B = 6
    oracle = om.test_init_(om.GPTOracle(3, 8, 256), seed=5)
    planes, _ = positions(B, seed=9)
    gen = torch.Generator().manual_seed(t)
    idx = torch.randint(0, 1929, (B, t), generator=gen)
    idx[0, -1] = 1928            # an ignored target inside the sequence
    rl, _, rt = oracle.forward_tokens(planes, idx, compute_loss=False)
    ra, rloss, _ = oracle.forward_tokens(planes, idx, compute_loss=True)
    m = models.GPT(models.GPTConfig(block_size=256, vocab_size=1929, n_layer=3, n_head=8, n_embd=256))
    m.load_state_dict(oracle.state_dict())
    logits, loss, targets = m.forward((planes.to(cuda), idx.to(cuda)))
    assert logits.shape == (B, 1, 1929) and loss is None and torch.equal(targets.cpu(), rt)
    assert rel_rms(logits.cpu(), rl) < 1e-2
    alll, loss, _ = m.forward((planes.to(cuda), idx.to(cuda)), compute_loss=True)
    assert alll.shape == (B, 64 + t, 1929)
    print("gpt T=%d: last rel-rms %.2e, all rel-rms %.2e, loss %.5f vs %.5f" % (64 + t, rel_rms(logits.cpu(), rl), rel_rms(alll.cpu(), ra), loss.item(), rloss.item()))
    assert rel_rms(alll.cpu(), ra) < 1e-2
    assert abs(loss.item() - rloss.item()) < 2e-3
    # the last row of the per-token logits is the last-token call; the first 64 rows do not depend on the move tokens
    assert torch.equal(alll[:, -1], logits[:, 0])
    base, _, _ = m.forward((planes.to(cuda), idx[:, :0].to(cuda)), compute_loss=True)
    assert torch.allclose(alll[:, :64], base, atol=1e-6, rtol=0)
    with pytest.raises(ValueError):
        m.forward((planes.to(cuda), torch.zeros(B, 193, dtype=torch.int64, device=cuda)))


def test_generate_cached_equals_teacher_forced_forward(cuda):
    """Greedy generation with cached keys/values: every step's logits equal the logits the full (uncached) forward
    gives at that position when it is fed the generated tokens, and every token is the arg-max of its step."""
    B, steps = 5, 70
    oracle = om.test_init_(om.GPTOracle(3, 8, 256), seed=6)
    planes, _ = positions(B, seed=4)
    m = models.GPT(models.GPTConfig(block_size=256, vocab_size=1929, n_layer=3, n_head=8, n_embd=256))
    m.load_state_dict(oracle.state_dict())
    seq, logits = m._engine.generate(planes.to(cuda), steps, T=0.0, rules=False, want_step_out=True, out_logits=True)
    assert seq.shape == (B, steps + 1) and bool((seq[:, 0] == 1924).all())
    assert torch.equal(seq[:, 1:], logits.argmax(-1))
    full = m._engine.forward_tokens(planes.to(cuda), seq[:, :steps].contiguous(), last=False, every=True)[1]
    err = rel_rms(logits.cpu(), full[:, 64:64 + steps].cpu())
    print("generate: cached vs recomputed logits rel-rms %.2e" % err)
    assert err < 3e-3
    # and against the fp32 oracle fed the same tokens
    ra, _, _ = oracle.forward_tokens(planes, seq[:, :steps].cpu(), compute_loss=True)
    assert rel_rms(logits.cpu(), ra[:, 64:64 + steps]) < 1e-2
    # the reference's entry points: full length, probabilities that sum to one, reproducible draws
    s1, p1 = m.generate_sequence(planes.to(cuda), T=1, seed=3)
    s2, _ = m.generate_sequence(planes.to(cuda), T=1, seed=3)
    s3, _ = m.generate_sequence(planes.to(cuda), T=1, seed=4)
    assert s1.shape == (B, 192) and p1.shape == (B, 191, 1929) and torch.equal(s1, s2) and not torch.equal(s1, s3)
    assert torch.allclose(p1.sum(-1), torch.ones(B, 191, device=cuda), atol=1e-4)
    assert bool((p1.gather(2, s1[:, 1:, None]) > 0).all())
    s0, p0 = m.generate_sequence_raw(planes.to(cuda), T=0)
    assert p0 is None and s0.shape == (B, 192)
    # the thinking-mode move picker built on it (model_bis.py:321-356)
    fen = "r1bq1rk1/2pp1ppp/p1n2n2/2b1p3/1pP1P3/1B1P1N2/PP3PPP/RNBQR1K1 b - c3 0 9"
    legal = {mv[:-1] if mv.endswith("n") else mv for mv in board.legal_moves(fen)}
    mv, probs = m.get_move_from_fen(fen, T=1, return_probs=True)
    assert mv in legal and abs(probs.sum().item() - 1) < 1e-4
    assert torch.equal((probs > 0).cpu(), torch.from_numpy(board.legal_move_mask(fen)).bool())
    with pytest.raises(ValueError):
        m.get_move_from_fen(fen, T=0)


def test_generate_replayed_graph_equals_plain_launches(cuda):
    """The recorded-and-replayed token step gives bit-identical sequences and per-step probabilities to plain
    launches: temperature sampling with the forced-token rules, on the default stream and on a side stream, twice
    in a row with a different length (the graph is recorded per call)."""
    B = 6
    oracle = om.test_init_(om.GPTOracle(3, 8, 256), seed=9)
    planes, _ = positions(B, seed=10)
    m = models.GPT(models.GPTConfig(block_size=256, vocab_size=1929, n_layer=3, n_head=8, n_embd=256))
    m.load_state_dict(oracle.state_dict())
    x = planes.to(cuda)
    for steps, stream in ((60, None), (33, torch.cuda.Stream()), (4, None)):
        out = {}
        for graph in (False, True):
            m._engine.set_decode_graph(graph)
            if stream is None:
                out[graph] = m._engine.generate(x, steps, T=1.0, seed=21, rules=True, want_step_out=True)
            else:
                stream.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(stream):
                    out[graph] = m._engine.generate(x, steps, T=1.0, seed=21, rules=True, want_step_out=True)
                stream.synchronize()
        torch.cuda.synchronize()
        assert torch.equal(out[False][0], out[True][0]), steps
        assert torch.equal(out[False][1], out[True][1]), steps
    m._engine.set_decode_graph(False)


def test_generate_folded_layernorm_equals_separate_kernels(cuda):
    """The token step folds the LayerNorm after the out-projection and after FFN-2 into the second pass of those
    K-sliced GEMMs; the profiling mode keeps the separate LayerNorm launches. Same step logits up to summation order."""
    B, steps = 4, 40
    oracle = om.test_init_(om.GPTOracle(3, 8, 256), seed=11)
    planes, _ = positions(B, seed=12)
    m = models.GPT(models.GPTConfig(block_size=256, vocab_size=1929, n_layer=3, n_head=8, n_embd=256))
    m.load_state_dict(oracle.state_dict())
    x = planes.to(cuda)
    seq_a, log_a = m._engine.generate(x, steps, T=0.0, rules=False, want_step_out=True, out_logits=True)
    m._engine.set_profiling(True)
    seq_b, log_b = m._engine.generate(x, steps, T=0.0, rules=False, want_step_out=True, out_logits=True)
    prof = m._engine.get_profile()
    m._engine.set_profiling(False)
    assert prof["layernorm"]["launches"] > (2 * 3 + 1) * (steps - 1)     # every norm of every step ran as its own launch
    # greedy decoding can part ways after a near-tie, so compare the steps up to the first differing token
    same = (seq_a == seq_b).all(0).cpu().tolist()
    upto = same.index(False) if False in same else steps + 1
    assert upto >= 10
    err = rel_rms(log_a[:, :upto - 1].cpu(), log_b[:, :upto - 1].cpu())
    print("folded vs separate LayerNorm: %d common steps, logits rel-rms %.2e" % (upto - 1, err))
    assert err < 2e-3


def test_generate_forced_tokens(cuda):
    """generate_sequence's bookkeeping (model_bis.py:252-259) on a model rigged to prefer end_variation: the sequences
    equal the rule application of the oracle to the arg-max of the recorded step logits."""
    B, steps = 3, 20
    oracle = om.test_init_(om.GPTOracle(2, 8, 256), seed=7)
    sd = oracle.state_dict()
    u = sd["transformer.ln_f.bias"].clone()
    sd["lm_head.weight"][1926] = 40.0 * u / u.pow(2).sum()
    sd["transformer.wte.weight"] = sd["lm_head.weight"]
    planes, _ = positions(B, seed=8)
    m = models.GPT(models.GPTConfig(block_size=256, vocab_size=1929, n_layer=2, n_head=8, n_embd=256))
    m.load_state_dict(sd)
    seq, logits = m._engine.generate(planes.to(cuda), steps, T=0.0, rules=True, want_step_out=True, out_logits=True)
    want = om.apply_generation_rules(logits.argmax(-1).cpu())
    assert torch.equal(seq.cpu(), want)
    row = seq[0].tolist()
    assert row.count(1926) >= 5 and 1925 in row
    i = row.index(1925)
    assert row[1:i].count(1926) == 5 and row[i + 2] == 1927


def test_empty_batch(cuda):
    """B = 0 gives empty outputs (what the reference's torch modules do), for the board forward and the token forward."""
    m = models.BT4Class(2, 256, 384, 8)
    pol, wdl = m(torch.zeros(0, 8, 8, 19, device=cuda))
    assert pol.shape == (0, 1858) and wdl.shape == (0, 3)
    g = models.GPT(models.GPTConfig(block_size=256, vocab_size=1929, n_layer=2, n_head=8, n_embd=256))
    logits, loss, _ = g.forward((torch.zeros(0, 8, 8, 19, device=cuda), torch.zeros(0, 3, dtype=torch.int64, device=cuda)))
    assert logits.shape == (0, 1, 1929) and loss is None
    assert m.evaluate_fens([], T=1.0)[0].shape == (0, 1858)


def test_gpt_fp8_vs_emulation(cuda):
    """The reference's own fp8 model is the GPT of model_fp8.py (te.Linear at :43,45,90,92, high-precision LayerNorm,
    attention and residual stream): the HIP fp8 path against the quantise->dequantise oracle with the same static scales."""
    L, H, Cm = 3, 8, 256
    oracle = om.test_init_(om.GPTOracle(L, H, Cm), seed=11)
    calib, _ = positions(64, seed=5)
    planes, mask = positions(64, seed=6)
    plan = om.Fp8Plan(L)
    plan.recording = True
    oracle.forward_last(calib, plan)
    plan.recording = False
    ref8 = oracle.forward_last(planes, plan)
    ref32 = oracle.forward_last(planes)
    m = models.GPT(models.GPTConfig(block_size=256, vocab_size=1929, n_layer=L, n_head=H, n_embd=Cm), fp8=True)
    m.load_state_dict(oracle.state_dict())
    m.calibrate(calib.to(cuda))
    own = m._engine.get_amax()[:, :4]
    want = plan.amax.numpy()[:, :4]
    print("gpt amax rel diff (own calibration vs oracle fp32):", np.abs(own / want - 1).max())
    assert np.abs(own / want - 1).max() < 0.05
    full = m._engine.get_amax()
    full[:, :4] = want
    m._engine.set_amax(full)
    pol = m.forward((planes.to(cuda), None))[0][:, 0].cpu()
    report("gpt fp8 vs fp8-emulation", pol, ref8, mask)
    report("gpt fp8 vs fp32", pol, ref32, mask)
    report("fp8-emulation vs fp32 (oracle only)", ref8, ref32, mask)
    assert rel_rms(pol, ref8) < 5e-2
    assert rel_rms(pol, ref32) < 2 * rel_rms(ref8, ref32) + 1e-2
