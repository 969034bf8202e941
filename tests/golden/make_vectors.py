"""Writes tests/golden/reference_vectors.npz by running the reference's own module code on the CPU.

Run from the repository root in a container that holds the reference checkout (default /root/reference):

    python tests/golden/make_vectors.py [reference_root]

The fixture holds outputs only. Weights and inputs are regenerated bit-identically by tests/golden/fill.py, so
neither the reference nor any of its text travels with the repository.

How the reference is loaded. Its model files import python-chess, zstandard and a CUDA device at module top
(model_bis.py:17-19, new_paradigm/value.py:19-21,35-41), none of which exist here, although the classes on the
forward path use torch alone. So this script does not import those modules: it parses each file, keeps the
class definitions it names (and, for value.py, the module-level default sizes of value.py:15-18), compiles those
syntax-tree nodes as they are and executes them in a namespace that holds torch. The one edit is a device
redirect for value.py: the string constant "cuda" becomes "cpu" (its constructors call .to("cuda")).
new_paradigm/attn.py needs no help and is imported whole.

What is written (all float32):
  gpt_last      GPT.forward((planes, idx[:, :0]))[0]                    model_bis.py:171-199   [B,1,1929]
  gpt_tok_last  GPT.forward((planes, idx))[0]                           same                    [B,1,1929]
  gpt_tok_rows, gpt_tok_loss  GPT.forward((planes, idx), compute_loss=True): logits[:, TOK_ROWS] and the loss
  gpt_generated GPT.generate_sequence(planes, T=0)[0] on rigged weights  model_bis.py:213-268   [B,block_size-64]
  attn_out      RelativeMultiHeadAttention2(x, x, x, pe)                new_paradigm/attn.py:491-533
  bt4_policy, bt4_value  BT4.forward(inp, compute_loss=True)[:2]        new_paradigm/value.py:155-212
  grpo_loss_kl_legal_logpdiff  ChessGRPOTrainer.compute_loss_bis(...): loss, mean KL, legal probability, avg_logp_diff
                                                                       grpo_refactored.py:322-372
  leela_mapping_black, leela_to_rl_*  the mirror table and map_leela_to_rl(policies, first_is_white)
                                                                       Leela/compare_policy.py:469-523
"""
import ast
import importlib.util
import math
import os
import sys
from dataclasses import dataclass

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
from fill import det_fill, fill_state_dict, rig_end_variation  # noqa: E402

# sizes of the fixture models (small, head size 32 so that the GPU library accepts them too)
GPT_CFG = dict(block_size=96, vocab_size=1929, n_layer=2, n_head=4, n_embd=128, dropout=0.0, bias=True)
GPT_B, GPT_T = 3, 7
TOK_ROWS = [0, 31, 63, 64, 70]   # rows of the all-token logits kept (the loss covers every row)
BT4_CFG = dict(num_layers=2, d_model=128, d_ff=192, num_heads=4)
BT4_B, BT4_S = 2, 2
ATTN_B = 3
GRPO_G, GRPO_B, GRPO_BETA, GRPO_LEGAL_W = 2, 2, 0.04, 0.1


def planes_input(name, shape):
    """Board-like planes: zeros and ones (about one in eight), last plane a fraction."""
    x = (det_fill(name, shape, 0.0, 1.0) < 0.125).astype(np.float32)
    x[..., 18] = det_fill(name + ".clock", shape[:-1], 0.0, 1.0)
    return x


def token_input(name, shape):
    return (det_fill(name, shape, 0.0, 1.0) * 1924).astype(np.int64)


class _Redirect(ast.NodeTransformer):
    def visit_Constant(self, node):
        return ast.copy_location(ast.Constant("cpu"), node) if node.value == "cuda" else node


def classes_of(path, names, namespace, redirect_cuda=False):
    tree = ast.parse(open(path).read(), filename=path)
    keep = []
    for node in tree.body:
        if isinstance(node, ast.ClassDef) and node.name in names:
            keep.append(node)
        elif isinstance(node, ast.Assign) and all(isinstance(t, ast.Name) and t.id in names for t in node.targets):
            keep.append(node)
    mod = ast.Module(body=keep, type_ignores=[])
    if redirect_cuda:
        mod = _Redirect().visit(mod)
    exec(compile(ast.fix_missing_locations(mod), path, "exec"), namespace)
    missing = [n for n in names if n not in namespace]
    assert not missing, "not found in %s: %s" % (path, missing)
    return namespace


def functions_of(path, class_name, names, namespace, redirect_cuda=False):
    """The named methods of one class, compiled as plain functions (first argument: whatever stands in for self)."""
    lines = open(path).read().split("\n")
    # Only the class is parsed: the script part of grpo_refactored.py uses an f-string form that needs Python 3.12.
    start = [i for i, l in enumerate(lines) if l.startswith("class " + class_name)][0]
    stop = [i for i in range(start + 1, len(lines)) if lines[i] and not lines[i][0].isspace() and not lines[i].startswith("#")]
    tree = ast.parse("\n" * start + "\n".join(lines[start:stop[0] if stop else len(lines)]), filename=path)
    cls = tree.body[0]
    mod = ast.Module(body=[n for n in cls.body if isinstance(n, ast.FunctionDef) and n.name in names], type_ignores=[])
    if redirect_cuda:
        mod = _Redirect().visit(mod)
    exec(compile(ast.fix_missing_locations(mod), path, "exec"), namespace)
    return namespace


def statements_of(path, names, namespace):
    """Module-level functions, assignments to the named variables, and loops that fill one of them."""
    tree = ast.parse(open(path).read(), filename=path)
    keep = []
    for node in tree.body:
        if isinstance(node, ast.FunctionDef) and node.name in names:
            keep.append(node)
        elif isinstance(node, ast.Assign) and all(isinstance(t, ast.Name) and t.id in names for t in node.targets):
            keep.append(node)
        elif isinstance(node, ast.For) and any(isinstance(n, ast.Subscript) and isinstance(n.value, ast.Name) and
                                               n.value.id in names and isinstance(n.ctx, ast.Store) for n in ast.walk(node)):
            keep.append(node)
    exec(compile(ast.fix_missing_locations(ast.Module(body=keep, type_ignores=[])), path, "exec"), namespace)
    return namespace


def grpo_inputs():
    """new_logits, ref_logits [G,B,256,1929], advantages [G,B], sampled sequences [G,B,192] (an `end` token at a
    different place in each, none in one of them), legal masks [G,B,1929]."""
    G, B = GRPO_G, GRPO_B
    new_logits = det_fill("grpo.new", (G, B, 256, 1929), -3.0, 3.0)
    ref_logits = (new_logits + det_fill("grpo.delta", (G, B, 256, 1929), -1.0, 1.0)).astype(np.float32)
    adv = det_fill("grpo.adv", (G, B), -1.5, 1.5)
    seqs = token_input("grpo.seq", (G, B, 192))
    for i, at in enumerate([5, 191, None, 60][: G * B]):
        if at is not None:
            seqs.reshape(-1, 192)[i, at] = 1927
    legal = (det_fill("grpo.legal", (G, B, 1929), 0.0, 1.0) < 0.02).astype(np.float32)
    return new_logits, ref_logits, adv, seqs, legal


def load_filled(module):
    sd = module.state_dict()
    filled = fill_state_dict({k: tuple(v.shape) for k, v in sd.items() if k != "pe"})
    module.load_state_dict({k: torch.from_numpy(v) for k, v in filled.items()}, strict=False)
    return module.eval()


def main(ref):
    base = dict(torch=torch, nn=nn, F=F, math=math, dataclass=dataclass, np=np)
    out = {}
    with torch.no_grad():
        # ---- GPT (model_bis.py) on top of the stem of utils/fen_encoder.py
        ns = classes_of(os.path.join(ref, "utils", "fen_encoder.py"), ["MaGating", "FenEncoder"], dict(base))
        ns = classes_of(os.path.join(ref, "model_bis.py"),
                        ["LayerNorm", "CausalSelfAttention", "MLP", "Block", "GPTConfig", "GPT"], ns)
        gpt = load_filled(ns["GPT"](ns["GPTConfig"](**GPT_CFG)))
        planes = torch.from_numpy(planes_input("gpt.planes", (GPT_B, 8, 8, 19)))
        idx = torch.from_numpy(token_input("gpt.idx", (GPT_B, GPT_T)))
        out["gpt_last"] = gpt((planes, idx[:, :0]))[0].numpy()
        out["gpt_tok_last"] = gpt((planes, idx))[0].numpy()
        logits, loss, _ = gpt((planes, idx), compute_loss=True)
        out["gpt_tok_rows"], out["gpt_tok_loss"] = logits[:, TOK_ROWS].numpy(), loss.numpy()
        # greedy generation with the forced-token rules, on a model rigged to prefer end_variation
        ns.update(start_think_index=1924, end_think_index=1925, end_variation_index=1926, end_index=1927)
        arrays = rig_end_variation(fill_state_dict({k: tuple(v.shape) for k, v in gpt.state_dict().items() if k != "pe"}))
        gpt.load_state_dict({k: torch.from_numpy(v) for k, v in arrays.items()}, strict=False)
        seq, probs = gpt.generate_sequence(planes, T=0)
        assert probs is None
        out["gpt_generated"] = seq.numpy()

        # ---- relative attention (new_paradigm/attn.py), imported whole
        spec = importlib.util.spec_from_file_location("ref_attn", os.path.join(ref, "new_paradigm", "attn.py"))
        attn_mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(attn_mod)
        C, H = BT4_CFG["d_model"], BT4_CFG["num_heads"]
        att = attn_mod.RelativeMultiHeadAttention2(C, H, 0)
        filled = fill_state_dict({"attention." + k: tuple(v.shape) for k, v in att.state_dict().items()})
        att.load_state_dict({k[len("attention."):]: torch.from_numpy(v) for k, v in filled.items()})
        x = torch.from_numpy(det_fill("attn.x", (ATTN_B, 64, C), -1.0, 1.0))
        pe = torch.from_numpy(det_fill("attn.pe", (1, 64, C), -1.0, 1.0)).expand(ATTN_B, -1, -1)
        out["attn_out"] = att.eval()(x, x, x, pe).numpy()

        # ---- BT4 (new_paradigm/value.py)
        ns = dict(base, RelativeMultiHeadAttention2=attn_mod.RelativeMultiHeadAttention2)
        ns = classes_of(os.path.join(ref, "new_paradigm", "value.py"),
                        ["num_layers", "d_model", "d_ff", "num_heads", "MaGating", "EncoderLayer",
                         "AbsolutePositionalEncoder", "ValueHead", "BT4"], ns, redirect_cuda=True)
        bt4 = load_filled(ns["BT4"](**BT4_CFG))
        planes = torch.from_numpy(planes_input("bt4.planes", (BT4_B, BT4_S, 8, 8, 19)))
        targets = torch.zeros(BT4_B, BT4_S, dtype=torch.int64)
        values = torch.zeros(BT4_B, BT4_S, 1, dtype=torch.int64)
        res = bt4([planes, targets, None, values], compute_loss=True)
        out["bt4_policy"], out["bt4_value"] = res[0].numpy(), res[1].numpy()
        assert torch.equal(bt4([planes]), res[0])

        # ---- GRPO scoring terms (grpo_refactored.py:322-372), the method run with a stand-in for `self`
        import types
        ns = functions_of(os.path.join(ref, "grpo_refactored.py"), "ChessGRPOTrainer", ["compute_loss_bis"],
                          dict(base, end_index=1927, print=lambda *a, **k: None), redirect_cuda=True)
        me = types.SimpleNamespace(beta=GRPO_BETA, config={"legal_loss_weight": GRPO_LEGAL_W})
        new_logits, ref_logits, adv, seqs, legal = (torch.from_numpy(a) for a in grpo_inputs())
        loss, mean_kl, legal_prob = ns["compute_loss_bis"](me, new_logits, ref_logits, adv, seqs, legal)
        out["grpo_loss_kl_legal_logpdiff"] = np.array([loss.item(), mean_kl.item(), legal_prob.item(), me.avg_logp_diff.item()])

    # ---- the 1858 -> 1929 move remap tables (Leela/compare_policy.py:469-523)
    ns = statements_of(os.path.join(ref, "Leela", "compare_policy.py"),
                       ["policy_index_leela", "policy_index", "policy_index_leela_size", "policy_index_size",
                        "mirror_uci_string", "policy_dict", "mapping_black", "mapping_white", "map_leela_to_rl"], dict(base))
    out["leela_mapping_black"] = ns["mapping_black"].astype(np.float32)
    pol = det_fill("leela.policies", (4, 1858), 0.0, 1.0)
    out["leela_to_rl_white_first"] = ns["map_leela_to_rl"](pol, True)
    out["leela_to_rl_black_first"] = ns["map_leela_to_rl"](pol, False)

    path = os.path.join(HERE, "reference_vectors.npz")
    np.savez_compressed(path, **{k: np.asarray(v, dtype=np.float32) for k, v in out.items()})
    for k, v in out.items():
        print(k, np.asarray(v).shape, float(np.abs(v).mean()))
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
