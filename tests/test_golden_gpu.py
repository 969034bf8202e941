"""The HIP forward passes (through the C ABI) against output vectors of the reference's own module code
(tests/golden/reference_vectors.npz): no oracle in between. 16-bit activations, so the tolerance is the bf16 bar
of the whole-model tests: relative RMS error of the logits under 2e-2 (bf16) / 4e-3 (f16), WDL within 1e-2."""
import os
import sys

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import make_vectors as mv  # noqa: E402
from fill import det_fill, fill_state_dict  # noqa: E402

from chessrl_amd import models  # noqa: E402

pytestmark = pytest.mark.gpu
GOLD = np.load(os.path.join(HERE, "golden", "reference_vectors.npz"))


def rel_rms(got, want):
    want = torch.from_numpy(np.asarray(want))
    return ((got.float().cpu() - want).pow(2).mean().sqrt() / want.pow(2).mean().sqrt()).item()


def load_filled(m):
    sd = m.state_dict()
    arrays = fill_state_dict({k: tuple(v.shape) for k, v in sd.items() if k != "pe"})
    tensors = {k: torch.from_numpy(v) for k, v in arrays.items()}
    if "pe" in sd:
        tensors["pe"] = sd["pe"]
    m.load_state_dict(tensors)
    return m


def test_gpt_against_reference_vectors(cuda):
    c = mv.GPT_CFG
    m = load_filled(models.GPT(models.GPTConfig(**c)))
    planes = torch.from_numpy(mv.planes_input("gpt.planes", (mv.GPT_B, 8, 8, 19))).to(cuda)
    idx = torch.from_numpy(mv.token_input("gpt.idx", (mv.GPT_B, mv.GPT_T))).to(cuda)
    last = m.forward((planes, idx[:, :0]))[0]
    tok_last = m.forward((planes, idx))[0]
    tok_all, loss, _ = m.forward((planes, idx), compute_loss=True)
    errs = (rel_rms(last, GOLD["gpt_last"]), rel_rms(tok_last, GOLD["gpt_tok_last"]),
            rel_rms(tok_all[:, mv.TOK_ROWS], GOLD["gpt_tok_rows"]))
    print("gpt vs reference vectors: rel-rms %.2e %.2e %.2e, loss %.5f vs %.5f" % (errs + (loss.item(), float(GOLD["gpt_tok_loss"]))))
    assert max(errs) < 2e-2
    assert abs(loss.item() - float(GOLD["gpt_tok_loss"])) < 5e-3
    want = torch.from_numpy(GOLD["gpt_last"])[:, 0]
    assert torch.equal(last[:, 0].float().cpu().argmax(-1), want.argmax(-1))


@pytest.mark.parametrize("act", ["bf16", "f16"])
def test_bt4_against_reference_vectors(cuda, act):
    c = mv.BT4_CFG
    m = load_filled(models.BT4(c["num_layers"], c["d_model"], c["d_ff"], c["num_heads"], act_dtype=act))
    planes = torch.from_numpy(mv.planes_input("bt4.planes", (mv.BT4_B, mv.BT4_S, 8, 8, 19))).to(cuda)
    pol = m.forward([planes])
    assert pol.shape == (mv.BT4_B, mv.BT4_S, 1929)
    _, wdl = m.evaluate(planes.reshape(-1, 8, 8, 19))
    e = rel_rms(pol, GOLD["bt4_policy"])
    w = (wdl.float().cpu() - torch.from_numpy(GOLD["bt4_value"]).reshape(-1, 3)).abs().max().item()
    print("bt4 %s vs reference vectors: policy rel-rms %.2e, wdl max-abs %.2e" % (act, e, w))
    assert e < (2e-2 if act == "bf16" else 4e-3)
    assert w <= (1e-2 if act == "bf16" else 2e-3)


def test_leela_to_rl_kernel_against_reference_vectors(cuda):
    import ctypes as C
    from chessrl_amd._lib import check, lib
    pol = torch.from_numpy(det_fill("leela.policies", (4, 1858), 0.0, 1.0)).to(cuda)
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    for first_white, key in ((True, "leela_to_rl_white_first"), (False, "leela_to_rl_black_first")):
        wtm = torch.tensor([(r % 2 == 0) == first_white for r in range(4)], dtype=torch.uint8, device=cuda)
        dst = torch.full((4, 1929), 7.0, device=cuda)
        check(lib().crl_leela_to_rl(C.c_void_p(pol.data_ptr()), 1858, C.c_void_p(dst.data_ptr()), 1929,
                                    C.c_void_p(wtm.data_ptr()), 4, st), "crl_leela_to_rl")
        assert np.array_equal(dst.cpu().numpy(), GOLD[key])


def test_grpo_terms_against_reference_vectors(cuda):
    """crl_token_scores' three outputs, assembled the way ChessGRPOTrainer.compute_loss_bis (grpo_refactored.py:322-372)
    assembles its own: mean of the masked per-token KL, and the signed mean log-probability difference."""
    G, B = mv.GRPO_G, mv.GRPO_B
    new_logits, ref_logits, adv, seqs, _ = (torch.from_numpy(a).to(cuda) for a in mv.grpo_inputs())
    new_l = new_logits[:, :, 63:-1].reshape(-1, 1929).contiguous()
    ref_l = ref_logits[:, :, 63:-1].reshape(-1, 1929).contiguous()
    logp, rlogp, kl = models.token_scores(new_l, seqs.reshape(-1), ref_l, want_kl=True)
    logp, rlogp, kl = (t.view(G, B, 192) for t in (logp, rlogp, kl))
    pos = torch.arange(192, device=cuda)
    first = torch.where(seqs == 1927, pos.expand_as(seqs), 192).min(-1).values
    mask = (pos.view(1, 1, -1) <= first.unsqueeze(-1)).float()
    mean_kl = ((kl * mask).sum(-1) / mask.sum(-1)).mean().item()
    a = adv.view(G, B, 1)
    diff = ((a > 0) * (logp - rlogp) + (a < 0) * (rlogp - logp)).mean().item()
    per_token = -(a - mv.GRPO_BETA * kl)     # exp(new - new.detach()) is one
    loss_without_legal_term = ((per_token * mask).sum(-1) / mask.sum(-1)).mean().item()
    want_loss, want_kl, _, want_diff = GOLD["grpo_loss_kl_legal_logpdiff"].tolist()
    print("grpo terms: mean kl %.6f vs %.6f, logp diff %.6f vs %.6f" % (mean_kl, want_kl, diff, want_diff))
    assert abs(mean_kl - want_kl) < 1e-5 * max(1.0, abs(want_kl))
    assert abs(diff - want_diff) < 1e-5
    # the remaining term of the loss (KL of the played move's distribution to the legal mask) is the caller's
    assert loss_without_legal_term < want_loss + 1e-4
