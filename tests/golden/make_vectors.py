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
  attn_out      RelativeMultiHeadAttention2(x, x, x, pe)                new_paradigm/attn.py:491-533
  bt4_policy, bt4_value  BT4.forward(inp, compute_loss=True)[:2]        new_paradigm/value.py:155-212
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
from fill import det_fill, fill_state_dict  # noqa: E402

# sizes of the fixture models (small, head size 32 so that the GPU library accepts them too)
GPT_CFG = dict(block_size=96, vocab_size=1929, n_layer=2, n_head=4, n_embd=128, dropout=0.0, bias=True)
GPT_B, GPT_T = 3, 7
TOK_ROWS = [0, 31, 63, 64, 70]   # rows of the all-token logits kept (the loss covers every row)
BT4_CFG = dict(num_layers=2, d_model=128, d_ff=192, num_heads=4)
BT4_B, BT4_S = 2, 2
ATTN_B = 3


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

    path = os.path.join(HERE, "reference_vectors.npz")
    np.savez_compressed(path, **{k: np.asarray(v, dtype=np.float32) for k, v in out.items()})
    for k, v in out.items():
        print(k, np.asarray(v).shape, float(np.abs(v).mean()))
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
