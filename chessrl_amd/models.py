"""Python surface of the reference models on top of the HIP library.

GPTConfig / GPT keep the constructor, state-dict keys and inference methods of
model_bis.py:115-398 for the 64-token ("no thinking") forward; BT4 keeps those of
new_paradigm/value.py:121-400; BT4Class is the benchmark's BT4-class encoder. All
compute runs in libchessrl_amd.so; torch only owns device memory and streams.
"""
import ctypes as C
import math
from collections import OrderedDict
from dataclasses import dataclass

import numpy as np
import torch

from . import _lib, board
from ._lib import check, lib
from .vocab import policy_index, policy_leela

VOCAB_RL, VOCAB_LEELA = _lib.VOCAB_RL, _lib.VOCAB_LEELA


def _stream_ptr():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def _lin_shapes(d, name, out, inp, bias=True):
    d[name + ".weight"] = (out, inp)
    if bias:
        d[name + ".bias"] = (out,)


def _ln_shapes(d, name, n):
    d[name + ".weight"] = (n,)
    d[name + ".bias"] = (n,)


def gpt_shapes(n_layer, n_embd, block_size=256, vocab_size=VOCAB_RL):
    """State-dict keys and shapes of model_bis.GPT (model_bis.py:132-146)."""
    C_ = n_embd
    d = OrderedDict()
    _lin_shapes(d, "FenEncoder.linear1", C_, 19)
    _ln_shapes(d, "FenEncoder.layernorm1", C_)
    d["FenEncoder.ma_gating.a"] = (64, C_)
    d["FenEncoder.ma_gating.b"] = (64, C_)
    d["transformer.wte.weight"] = (vocab_size, C_)
    for i in range(n_layer):
        p = "transformer.h.%d." % i
        _ln_shapes(d, p + "ln_1", C_)
        _lin_shapes(d, p + "attn.c_attn", 3 * C_, C_)
        _lin_shapes(d, p + "attn.c_proj", C_, C_)
        _ln_shapes(d, p + "ln_2", C_)
        _lin_shapes(d, p + "mlp.c_fc", 4 * C_, C_)
        _lin_shapes(d, p + "mlp.c_proj", C_, 4 * C_)
    _ln_shapes(d, "transformer.ln_f", C_)
    d["lm_head.weight"] = (vocab_size, C_)
    d["pe"] = (block_size, C_)
    return d


def bt4_shapes(num_layers, d_model, d_ff, num_heads, bt4class=False, compress=32, hidden=256, gen=256):
    """State-dict keys and shapes of new_paradigm/value.py BT4 (value.py:129-152,423-425);
    with bt4class=True the BT4-class extension (smolgen, promotion offsets, no dense policy map)."""
    C_, F_, H = d_model, d_ff, num_heads
    d = OrderedDict()
    for i in range(num_layers):
        p = "layers.%d." % i
        for n in ("query_proj", "key_proj", "value_proj"):
            _lin_shapes(d, p + "attention." + n, C_, C_)
        if not bt4class:
            d[p + "attention.pos_proj.weight"] = (C_, C_)
            d[p + "attention.u_bias"] = (H, C_ // H)
            d[p + "attention.v_bias"] = (H, C_ // H)
        _lin_shapes(d, p + "attention.out_proj", C_, C_)
        if bt4class:
            d[p + "smolgen.compress.weight"] = (compress, C_)
            _lin_shapes(d, p + "smolgen.hidden", hidden, 64 * compress)
            _ln_shapes(d, p + "smolgen.hidden_ln", hidden)
            _lin_shapes(d, p + "smolgen.gen_from", H * gen, hidden)
            _ln_shapes(d, p + "smolgen.gen_from_ln", H * gen)
        _ln_shapes(d, p + "norm1", C_)
        _ln_shapes(d, p + "norm2", C_)
        _lin_shapes(d, p + "ff1", F_, C_)
        _lin_shapes(d, p + "ff2", C_, F_)
    if bt4class:
        d["smol_weight_gen.weight"] = (4096, gen)
    _lin_shapes(d, "linear1", C_, 19)
    _ln_shapes(d, "layernorm1", C_)
    _lin_shapes(d, "policy_tokens_lin", C_, C_)
    _lin_shapes(d, "queries_pol", C_, C_)
    _lin_shapes(d, "keys_pol", C_, C_)
    d["ma_gating.a"] = (64, C_)
    d["ma_gating.b"] = (64, C_)
    if bt4class:
        d["promotion_offsets.weight"] = (4, C_)
    else:
        d["policy_head.weight"] = (VOCAB_RL, 4096)
    _lin_shapes(d, "value_head.dense1", 128, C_)
    _lin_shapes(d, "value_head.dense2", 128, 128 * 64)
    _lin_shapes(d, "value_head.dense3", 3, 128)
    return d


def _default_init(shapes, seed, n_layer=None):
    """normal(0, 0.02) weights, zero biases, LayerNorm at identity, gating a=0/b=1
    (model_bis.py:163-169); c_proj weights use std 0.02/sqrt(2L) (model_bis.py:153-155)."""
    g = torch.Generator().manual_seed(seed)
    sd = OrderedDict()
    for k, shp in shapes.items():
        if k == "pe":
            continue
        if k.endswith("ma_gating.a"):
            t = torch.zeros(shp)
        elif k.endswith("ma_gating.b"):
            t = torch.ones(shp)
        elif k.endswith("u_bias") or k.endswith("v_bias"):
            bound = math.sqrt(6.0 / (shp[0] + shp[1]))
            t = torch.empty(shp).uniform_(-bound, bound, generator=g)
        elif len(shp) == 2:
            std = 0.02 / math.sqrt(2 * n_layer) if (k.endswith("c_proj.weight") and n_layer) else 0.02
            t = torch.empty(shp).normal_(0.0, std, generator=g)
        elif k.endswith(".bias"):
            t = torch.zeros(shp)
        else:
            t = torch.ones(shp)
        sd[k] = t
    return sd


def token_scores(logits, target=None, ref_logits=None, ignore_index=-100, want_kl=False):
    """Row-wise log-softmax statistics of cuda float32 logits [rows, V] through the library's kernel:
    returns (logp [rows] of `target` or None, ref_logp or None, kl(softmax(logits) || softmax(ref_logits)) or None)."""
    rows, V = logits.shape
    assert logits.stride(1) == 1 and (ref_logits is None or ref_logits.stride(1) == 1)
    dev = logits.device
    logp = torch.empty(rows, dtype=torch.float32, device=dev) if target is not None else None
    rlogp = torch.empty(rows, dtype=torch.float32, device=dev) if (target is not None and ref_logits is not None) else None
    kl = torch.empty(rows, dtype=torch.float32, device=dev) if (want_kl and ref_logits is not None) else None
    tgt = target.to(torch.int64).contiguous() if target is not None else None
    check(lib().crl_token_scores(_ptr(logits), logits.stride(0), _ptr(ref_logits), ref_logits.stride(0) if ref_logits is not None else 0,
                                 _ptr(tgt), rows, V, int(ignore_index), _ptr(logp), _ptr(rlogp), _ptr(kl), _stream_ptr()), "crl_token_scores")
    return logp, rlogp, kl


def cross_entropy(logits, targets, ignore_index=-100):
    """F.cross_entropy(logits, targets, ignore_index=...) (mean over the rows that count) on the device."""
    tgt = targets.to(torch.int64).contiguous()
    logp, _, _ = token_scores(logits, tgt, ignore_index=ignore_index)
    out = torch.empty(1, dtype=torch.float32, device=logits.device)
    check(lib().crl_masked_nll_mean(_ptr(logp), _ptr(tgt), int(ignore_index), logits.shape[0], _ptr(out), _stream_ptr()), "crl_masked_nll_mean")
    return out[0]


class _Engine:
    """Owns one crl_model handle."""

    def __init__(self, arch, n_layer, d_model, n_head, d_ff, fp8=False, micro_batch=0, stream_f32=None,
                 head_dtype=None, act_dtype="bf16", compress=32, hidden=256, gen=256, ln_fold=None, norm_rms=False,
                 fp8_lm_head=None):
        cfg = _lib.ModelConfig()
        cfg.arch, cfg.n_layer, cfg.d_model, cfg.n_head, cfg.d_ff = arch, n_layer, d_model, n_head, d_ff
        cfg.fp8 = 1 if fp8 else 0
        cfg.micro_batch = micro_batch
        tri = lambda v: 0 if v is None else 1 if v else -1     # None = the library's default
        cfg.stream_f32 = tri(stream_f32)
        cfg.ln_fold = tri(ln_fold)
        cfg.fp8_lm_head = tri(fp8_lm_head)
        cfg.norm_rms = 1 if norm_rms else 0
        cfg.act_dtype = _lib.F16 if act_dtype in ("f16", "fp16") else _lib.BF16
        cfg.head_dtype = cfg.act_dtype if head_dtype is None else _lib.F16 if head_dtype in ("f16", "fp16") else _lib.BF16
        cfg.smolgen_compress, cfg.smolgen_hidden, cfg.smolgen_gen = compress, hidden, gen
        self.cfg = cfg
        self.n_layer = n_layer
        self.fp8 = bool(fp8)
        h = C.c_void_p()
        check(lib().crl_model_create(C.byref(cfg), C.byref(h)), "crl_model_create")
        self.handle = h
        self.vocab = lib().crl_model_vocab(h)
        self.ready = False

    def __del__(self):
        h = getattr(self, "handle", None)
        if h:
            try:
                lib().crl_model_destroy(h)
            except Exception:
                pass
            self.handle = None

    def expected_keys(self):
        out, i, n = [], 0, C.c_int64()
        while True:
            k = lib().crl_model_expected_key(self.handle, i, C.byref(n))
            if k is None:
                return out
            out.append((k.decode(), n.value))
            i += 1

    def load(self, sd):
        for k, _ in self.expected_keys():
            if k not in sd:
                raise KeyError("state dict lacks %r" % k)
            t = sd[k].detach().to("cpu", torch.float32).contiguous()
            check(lib().crl_model_set_weight(self.handle, k.encode(), C.c_void_p(t.data_ptr()), t.numel()), "crl_model_set_weight(%s)" % k)
        self.ready = False

    def finalize(self):
        if not torch.cuda.is_available():
            raise _lib.CrlError("no GPU: the forward pass has no CPU fallback")
        check(lib().crl_model_finalize(self.handle), "crl_model_finalize")
        self.ready = True

    def calibrate(self, planes):
        if not self.ready:
            self.finalize()
        planes = _as_planes(planes)
        check(lib().crl_model_calibrate(self.handle, _ptr(planes), planes.shape[0], _stream_ptr()), "crl_model_calibrate")

    def get_amax(self, head=None):
        """Activation amax table [n_layer, 5]; with head=True [n_layer + 1, 5], whose last row starts with the amax
        of lm_head's input (GPT64) or with the amax of the trunk output and of the policy tokens (BT4-class: the inputs
        of its e4m3 head linears). head=None picks the full table for the models whose heads run in e4m3 (a model that
        receives the short table keeps its heads in 16 bits) and the short one otherwise."""
        if head is None:
            head = self.fp8 and (self.cfg.arch == _lib.ARCH_GPT64 or (self.cfg.arch == _lib.ARCH_BT4CLASS and self.cfg.fp8_lm_head > 0))
        rows = self.n_layer + (1 if head else 0)
        a = np.zeros(rows * 5, np.float32)
        check(lib().crl_model_get_amax(self.handle, a.ctypes.data, a.size), "crl_model_get_amax")
        return a.reshape(rows, 5)

    def set_amax(self, a):
        a = np.ascontiguousarray(np.asarray(a, np.float32).reshape(-1))
        check(lib().crl_model_set_amax(self.handle, a.ctypes.data, a.size), "crl_model_set_amax")

    def forward(self, planes, want_wdl=True, out_policy=None, out_wdl=None):
        """planes: cuda float32 [B,64,19] (any shape with 64*19 trailing elements per position)."""
        if not self.ready:
            self.finalize()
        planes = _as_planes(planes)
        B = planes.shape[0]
        pol = out_policy if out_policy is not None else torch.empty((B, self.vocab), dtype=torch.float32, device=planes.device)
        wdl = None
        if want_wdl and self.cfg.arch != _lib.ARCH_GPT64:
            wdl = out_wdl if out_wdl is not None else torch.empty((B, 3), dtype=torch.float32, device=planes.device)
        check(lib().crl_model_forward(self.handle, _ptr(planes), B, _ptr(pol), _ptr(wdl), _stream_ptr()), "crl_model_forward")
        return pol, wdl

    def forward_compact(self, ids, flags, want_wdl=True):
        if not self.ready:
            self.finalize()
        B = ids.shape[0]
        pol = torch.empty((B, self.vocab), dtype=torch.float32, device=ids.device)
        wdl = torch.empty((B, 3), dtype=torch.float32, device=ids.device) if (want_wdl and self.cfg.arch != _lib.ARCH_GPT64) else None
        check(lib().crl_model_forward_compact(self.handle, _ptr(ids.contiguous()), _ptr(flags.contiguous()), B, _ptr(pol), _ptr(wdl), _stream_ptr()),
              "crl_model_forward_compact")
        return pol, wdl

    def forward_tokens(self, planes, idx, last=True, every=False):
        """CRL_ARCH_GPT64 with move tokens idx [B,t] (cuda int64): (logits of the last token [B,V] or None,
        logits of every token [B,64+t,V] or None)."""
        if not self.ready:
            self.finalize()
        planes = _as_planes(planes)
        B, t = planes.shape[0], idx.shape[1]
        lastl = torch.empty((B, self.vocab), dtype=torch.float32, device=planes.device) if last else None
        alll = torch.empty((B, 64 + t, self.vocab), dtype=torch.float32, device=planes.device) if every else None
        check(lib().crl_model_forward_tokens(self.handle, _ptr(planes), _ptr(idx) if t else None, B, t, _ptr(lastl), _ptr(alll), _stream_ptr()),
              "crl_model_forward_tokens")
        return lastl, alll

    def generate(self, planes, steps, T=1.0, seed=0, rules=True, want_step_out=False, out_logits=False):
        """CRL_ARCH_GPT64 sequence generation with cached keys/values: (sequences [B, steps+1] int64,
        per-step probabilities or logits [B, steps, V] or None)."""
        if not self.ready:
            self.finalize()
        planes = _as_planes(planes)
        B = planes.shape[0]
        seq = torch.empty((B, steps + 1), dtype=torch.int64, device=planes.device)
        out = torch.empty((B, steps, self.vocab), dtype=torch.float32, device=planes.device) if want_step_out else None
        check(lib().crl_model_generate(self.handle, _ptr(planes), B, int(steps), float(T), int(seed) & (2 ** 64 - 1), 1 if rules else 0,
                                       _ptr(seq), _ptr(out), 1 if out_logits else 0, _stream_ptr()), "crl_model_generate")
        return seq, out

    def evaluate_fens(self, fens, T=1.0, chunk=4096, want_probs=True, want_wdl=True, threads=0):
        """FEN strings -> (probs [n,V] or None, wdl logits [n,3] or None, best move index [n]) as CPU tensors.
        Host encoding, upload and device work of consecutive chunks overlap inside the library."""
        if not self.ready:
            self.finalize()
        n = len(fens)
        has_wdl = want_wdl and self.cfg.arch != _lib.ARCH_GPT64
        probs = torch.empty((n, self.vocab), dtype=torch.float32) if want_probs else None
        wdl = torch.empty((n, 3), dtype=torch.float32) if has_wdl else None
        best = torch.empty((n,), dtype=torch.int32)
        arr = _lib.str_array(fens)
        check(lib().crl_model_evaluate_fens(self.handle, arr, n, int(chunk), float(T), _ptr(probs), _ptr(wdl), _ptr(best), int(threads)),
              "crl_model_evaluate_fens")
        return probs, wdl, best

    def search_1ply(self, fens, T=0.0, seed=0, chunk=4096, want_values=False, threads=0):
        """Batched 1-ply value search: (best move per root, and with want_values the per-root (moves, values) lists)."""
        if not self.ready:
            self.finalize()
        n = len(fens)
        arr = _lib.str_array(fens)
        best = C.create_string_buffer(max(n, 1) * 6)
        counts = (C.c_int32 * max(n, 1))()
        cap = 256 * n if want_values else 0
        mv = C.create_string_buffer(max(cap, 1) * 6) if want_values else None
        vals = torch.empty((max(cap, 1),), dtype=torch.float32) if want_values else None
        check(lib().crl_model_search_1ply(self.handle, arr, n, int(chunk), float(T), int(seed) & (2 ** 64 - 1), best, counts,
                                          mv, _ptr(vals), cap, int(threads)), "crl_model_search_1ply")
        braw = best.raw                       # .raw copies the whole buffer: take it once
        moves = [braw[6 * i:6 * i + 6].split(b"\0")[0].decode() for i in range(n)]
        if not want_values:
            return moves
        mraw = mv.raw
        per_root, o = [], 0
        for i in range(n):
            k = counts[i]
            per_root.append(([mraw[6 * (o + c):6 * (o + c) + 6].split(b"\0")[0].decode() for c in range(k)], vals[o:o + k].clone()))
            o += k
        return moves, per_root

    def run_layers(self, x_in, first, last):
        """Encoder layers [first, last) on a caller-supplied layer input (cuda float32 [B,64,C]) -> output of layer
        last-1 (cuda float32 [B,64,C])."""
        if not self.ready:
            self.finalize()
        x_in = x_in.to(torch.float32).contiguous()
        out = torch.empty_like(x_in)
        check(lib().crl_model_run_layers(self.handle, _ptr(x_in), x_in.shape[0], int(first), int(last), _ptr(out), _stream_ptr()),
              "crl_model_run_layers")
        return out

    def read_tensor(self, name, shape, dtype=torch.uint8, device="cuda"):
        """A workspace tensor as the last call left it (see crl_model_read_tensor)."""
        out = torch.empty(shape, dtype=dtype, device=device)
        check(lib().crl_model_read_tensor(self.handle, name.encode(), _ptr(out), out.numel() * out.element_size(), _stream_ptr()),
              "crl_model_read_tensor")
        return out

    def flops_per_position(self):
        return lib().crl_model_flops_per_position(self.handle)

    def set_profiling(self, on):
        check(lib().crl_model_set_profiling(self.handle, 1 if on else 0), "crl_model_set_profiling")

    def set_decode_graph(self, on):
        check(lib().crl_model_set_decode_graph(self.handle, 1 if on else 0), "crl_model_set_decode_graph")

    def get_profile(self):
        ms = (C.c_double * 6)()
        n = (C.c_int64 * 6)()
        fl = (C.c_double * 6)()
        check(lib().crl_model_get_profile(self.handle, ms, n, fl), "crl_model_get_profile")
        names = ("gemm_fp8", "attention", "layernorm", "embed", "policy_qk", "gemm_16bit")
        return {k: {"ms": ms[i], "launches": n[i], "flops": fl[i]} for i, k in enumerate(names)}


def _as_planes(planes):
    if not planes.is_cuda:
        raise _lib.CrlError("planes must live on the GPU (the forward pass has no CPU path)")
    if planes.dtype != torch.float32:
        planes = planes.float()
    return planes.reshape(-1, 64, 19).contiguous()


def masked_softmax(logits, mask=None, temperature=1.0, want_probs=True):
    """softmax((logits + (1-mask)*-999)/T) and the arg-max, on the GPU (model_bis.py:382-392)."""
    logits = logits.contiguous()
    B, V = logits.shape
    probs = torch.empty_like(logits) if want_probs else None
    am = torch.empty((B,), dtype=torch.int32, device=logits.device)
    if mask is not None:
        mask = mask.to(torch.uint8).contiguous()
    check(lib().crl_masked_softmax(_ptr(logits), V, _ptr(mask), V, _ptr(probs), V, _ptr(am), B, V, float(temperature), _stream_ptr()),
          "crl_masked_softmax")
    return probs, am


def leela_to_rl(logits1858, white_to_move):
    """[B,1858] side-to-move-frame values -> [B,1929] policy_index slots (Leela/compare_policy.py:493-523)."""
    src = logits1858.contiguous()
    B = src.shape[0]
    dst = torch.empty((B, VOCAB_RL), dtype=torch.float32, device=src.device)
    wtm = white_to_move.to(torch.uint8).contiguous()
    check(lib().crl_leela_to_rl(_ptr(src), VOCAB_LEELA, _ptr(dst), VOCAB_RL, _ptr(wtm), B, _stream_ptr()), "crl_leela_to_rl")
    return dst


class _ModelBase:
    """Shared state-dict plumbing and the batched leaf-evaluation entry."""

    is_thinking_model = False

    def state_dict(self):
        return OrderedDict((k, v.clone()) for k, v in self._sd.items())

    def load_state_dict(self, sd, strict=True):
        # transformer_engine's Linear (model_fp8.py:43-45,90-92,140) stores its fp8 recipe state under '<module>._extra_state':
        # not weights, skipped. (The scales used here come from calibrate().)
        sd = OrderedDict((k, v) for k, v in sd.items() if not k.endswith("_extra_state"))
        missing = [k for k in self._shapes if k not in sd and k != "transformer.wte.weight"]
        unexpected = [k for k in sd if k not in self._shapes]
        if strict and (missing or unexpected):
            raise RuntimeError("load_state_dict: missing %s, unexpected %s" % (missing, unexpected))
        for k, shp in self._shapes.items():
            if k in sd:
                t = sd[k].detach().to("cpu", torch.float32)
                # pe may have more rows than used; lm_head / wte may carry padding rows behind the 1929 moves
                # (pretrain_fp8.py:16 trains with vocab_size 1936)
                grows = (k == "pe" and t.shape[0] >= 64) or (k in ("lm_head.weight", "transformer.wte.weight") and t.shape[0] >= VOCAB_RL)
                if tuple(t.shape) != tuple(shp) and not (grows and t.dim() == 2 and t.shape[1] == shp[1]):
                    raise RuntimeError("load_state_dict: %s has shape %s, expected %s" % (k, tuple(t.shape), tuple(shp)))
                self._sd[k] = t.clone()
        if "lm_head.weight" in self._sd:
            self._sd["transformer.wte.weight"] = self._sd["lm_head.weight"]
        self._engine.load(self._sd)
        return self

    def to(self, *a, **k):
        return self

    def eval(self):
        return self

    def parameters(self):
        return [v for k, v in self._sd.items() if k != "pe"]

    def calibrate(self, planes):
        """fp8: derive the static activation scales from a calibration batch."""
        self._engine.calibrate(planes)

    @torch.no_grad()
    def evaluate(self, planes, legal_mask=None, T=1.0, want_probs=False):
        """Batched leaf evaluation: planes [B,8,8,19] (cuda) -> (policy_logits [B,V], wdl_logits [B,3] or None).
        With want_probs the legal-masked softmax(./T) is returned in place of the raw logits."""
        pol, wdl = self._engine.forward(planes)
        if want_probs:
            pol, _ = masked_softmax(pol, legal_mask, T)
        return pol, wdl

    @torch.no_grad()
    def evaluate_fens(self, fens, T=1.0, chunk=4096, want_probs=True, want_wdl=True):
        """Leaf evaluation from FEN strings with everything host-side done in the library: parsing, encoding,
        legal masks, upload (overlapped with the device work of the previous chunk), masked softmax, download.
        Returns CPU tensors (probs [n,V] or None, wdl logits [n,3] or None, best legal move index [n])."""
        return self._engine.evaluate_fens(list(fens), T, chunk, want_probs, want_wdl)

    @torch.no_grad()
    def get_best_moves_value(self, fens, T=0.0, seed=0, return_values=False):
        """get_best_move_value (new_paradigm/value.py:356-400) for a list of positions in one call: every child of
        every root goes through the library's chunked pipeline. Returns the chosen move per root ('' where a root has
        no legal move) and, with return_values, per root (moves, value of each move for the side to move)."""
        return self._engine.search_1ply(list(fens), T=T, seed=seed, want_values=return_values)

    def graphed_evaluator(self, batch, T=1.0, device="cuda"):
        """Leaf evaluation for a fixed batch size captured in a HIP graph (launch-bound small batches)."""
        return GraphedEvaluator(self, batch, T, device)

    def _sample(self, logits_row, mask_row, T):
        probs, am = masked_softmax(logits_row, mask_row, T, want_probs=True)
        if T == 0:
            return int(am.item()), probs
        return int(torch.multinomial(probs, num_samples=1).item()), probs


class GraphedEvaluator:
    """forward + legal-masked softmax for one fixed batch size, recorded once into a HIP graph and
    replayed per call. The ~200 kernel launches of a forward pass dominate the latency of small
    batches (MCTS leaf evaluation); a replay issues them as one graph launch. The library calls
    record no memset nodes (flags and scratch are cleared by kernels)."""

    def __init__(self, model, batch, T=1.0, device="cuda"):
        eng = model._engine
        if not eng.ready:
            eng.finalize()
        self.batch, self.T = batch, float(T)
        self.planes = torch.zeros((batch, 64, 19), dtype=torch.float32, device=device)
        self.mask = torch.ones((batch, eng.vocab), dtype=torch.uint8, device=device)
        self.policy = torch.empty((batch, eng.vocab), dtype=torch.float32, device=device)
        self.probs = torch.empty_like(self.policy)
        self.argmax = torch.empty((batch,), dtype=torch.int32, device=device)
        self.wdl = torch.empty((batch, 3), dtype=torch.float32, device=device) if eng.cfg.arch != _lib.ARCH_GPT64 else None
        self._eng = eng
        self._run()                      # eager warm-up: allocates the workspace outside the capture
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self._run()

    def _run(self):
        self._eng.forward(self.planes, out_policy=self.policy, out_wdl=self.wdl)
        V = self._eng.vocab
        check(lib().crl_masked_softmax(_ptr(self.policy), V, _ptr(self.mask), V, _ptr(self.probs), V, _ptr(self.argmax),
                                       self.batch, V, self.T, _stream_ptr()), "crl_masked_softmax")

    @torch.no_grad()
    def __call__(self, planes, legal_mask=None):
        """planes [batch,8,8,19] on the GPU -> (probs [batch,V], wdl logits [batch,3] or None, argmax [batch]).
        The returned tensors are the evaluator's own buffers and are overwritten by the next call."""
        self.planes.copy_(planes.reshape(self.batch, 64, 19))
        if legal_mask is not None:
            self.mask.copy_(legal_mask)
        else:
            self.mask.fill_(1)
        self.graph.replay()
        return self.probs, self.wdl, self.argmax


@dataclass
class GPTConfig:
    block_size: int = 1024
    vocab_size: int = 50304
    n_layer: int = 6
    n_head: int = 12
    n_embd: int = 768
    dropout: float = 0.0
    bias: bool = True


class GPT(_ModelBase):
    """model_bis.GPT for the 64 board tokens (model_bis.py:125-199, 358-398)."""

    def __init__(self, config, fp8=False, micro_batch=0, stream_f32=True, head_dtype=None, act_dtype="bf16", seed=0,
                 norm_rms=False, fp8_lm_head=None):
        # vocab_size above 1929 (pretrain_fp8.py:16 pads to 1936 for the fp8 GEMM) adds rows to lm_head / wte that no
        # move uses: they are kept in the state dict, count towards the e4m3 weight scale, and the logits stay 1929 wide.
        if config.vocab_size < VOCAB_RL:
            raise ValueError("vocab_size must be at least %d (utils/vocab.py)" % VOCAB_RL)
        if not config.bias:
            raise ValueError("bias=False is not supported")
        self.config = config
        self._shapes = gpt_shapes(config.n_layer, config.n_embd, config.block_size, config.vocab_size)
        self._sd = _default_init(self._shapes, seed, config.n_layer)
        self._sd["transformer.wte.weight"] = self._sd["lm_head.weight"]
        from_pe = torch.zeros(config.block_size, config.n_embd)
        pos = torch.arange(config.block_size).unsqueeze(1)
        div = torch.exp(torch.arange(0, config.n_embd, 2).float() * (-math.log(10000.0) / config.n_embd))
        from_pe[:, 0::2] = torch.sin(pos * div)
        from_pe[:, 1::2] = torch.cos(pos * div)
        self._sd["pe"] = from_pe
        self._engine = _Engine(_lib.ARCH_GPT64, config.n_layer, config.n_embd, config.n_head, 4 * config.n_embd,
                               fp8=fp8, micro_batch=micro_batch, stream_f32=stream_f32, head_dtype=head_dtype, act_dtype=act_dtype,
                               norm_rms=norm_rms, fp8_lm_head=fp8_lm_head)
        self._engine.load(self._sd)

    def get_num_params(self, non_embedding=True):
        return sum(v.numel() for k, v in self._sd.items() if k not in ("pe", "transformer.wte.weight"))

    @torch.no_grad()
    def forward(self, batch, compute_loss=False):
        """batch = (planes [B,8,8,19], idx [B,t] int64 move tokens, t >= 0). Like model_bis.py:171-199 returns
        (logits, loss, targets): logits [B,1,1929] of the last token and loss None, or with compute_loss the logits
        of every token [B,64+t,1929] and the cross-entropy against the shifted targets (ignore_index 1928)."""
        planes, idx = batch[0], batch[1]
        B = _as_planes(planes).shape[0]
        dev = planes.device
        if idx is None:
            idx = torch.zeros((B, 0), dtype=torch.int64, device=dev)
        idx = idx.to(device=dev, dtype=torch.int64).contiguous()
        t = idx.shape[1]
        if 64 + t > self.config.block_size:
            raise ValueError("Cannot forward sequence of length %d, block size is %d" % (64 + t, self.config.block_size))
        targets = torch.cat((torch.full((B, 64), 1928, device=dev, dtype=torch.int64), idx), dim=1).roll(-1, dims=1)
        if not compute_loss:
            return self._engine.forward_tokens(planes, idx, last=True)[0].unsqueeze(1), None, targets
        logits = self._engine.forward_tokens(planes, idx, last=False, every=True)[1]
        loss = cross_entropy(logits.view(-1, logits.shape[-1]), targets.reshape(-1), ignore_index=1928)
        return logits, loss, targets

    __call__ = forward

    @torch.no_grad()
    def generate_sequence(self, board, T=1, seed=0):
        """model_bis.py:213-263: (sequences [B,192], probs [B,191,1929] or None for T == 0), with the forced
        </thinking> and end tokens. Keys and values of the prefix are cached instead of recomputed per token."""
        seq, probs = self._engine.generate(board, self.config.block_size - 65, T, seed, rules=True, want_step_out=T != 0)
        return seq, probs

    @torch.no_grad()
    def generate_sequence_raw(self, board, T=1, return_logits=False, seed=0):
        """model_bis.py:266-311: as generate_sequence without the forced tokens; the per-step output is the
        probabilities or, with return_logits, the logits."""
        return self._engine.generate(board, self.config.block_size - 65, T, seed, rules=False, want_step_out=T != 0, out_logits=return_logits)

    @torch.no_grad()
    def get_move_from_fen(self, fen, T=1, device="cuda", force_legal=True, return_probs=False, seed=0):
        """model_bis.py:321-356: generate a thinking sequence, take the logits of the step that produced the token
        before the first `end` (the last step's if there is none), mask them to the legal moves and sample.
        T must be positive (the reference divides by T and needs the per-step logits)."""
        if not T > 0:
            raise ValueError("get_move_from_fen needs T > 0")
        planes = board.encode_fens([fen]).to(device)
        seq, logits = self.generate_sequence_raw(planes, T=T, return_logits=True, seed=seed)
        ids = seq[0].tolist()
        end = policy_index.index("end")
        i = ids.index(end) if end in ids else len(ids) - 1
        row = logits[0, i - 2].unsqueeze(0)          # negative i-2 wraps like the reference's indexing
        mask = torch.from_numpy(board.legal_move_mask(fen)).to(device).unsqueeze(0) if force_legal else None
        idx, probs = self._sample(row, mask, T)
        move = policy_index[idx]
        return (move, probs[0]) if return_probs else move

    @torch.no_grad()
    def get_move_from_fen_no_thinking(self, fen, T=1, device="cuda", force_legal=True, return_probs=False):
        planes = board.encode_fens([fen]).to(device)
        logits, _ = self._engine.forward(planes)
        mask = torch.from_numpy(board.legal_move_mask(fen)).to(device).unsqueeze(0) if force_legal else None
        idx, probs = self._sample(logits, mask, T)
        move = policy_index[idx]
        return (move, probs[0]) if return_probs else move


class BT4(_ModelBase):
    """new_paradigm/value.py BT4 (value.py:121-400)."""

    def __init__(self, num_layers=10, d_model=512, d_ff=736, num_heads=8, fp8=False, micro_batch=0, head_dtype=None, act_dtype="bf16", seed=0,
                 stream_f32=None, norm_rms=False):
        self.num_layers, self.d_model = num_layers, d_model
        self._shapes = bt4_shapes(num_layers, d_model, d_ff, num_heads)
        self._sd = _default_init(self._shapes, seed)
        self._engine = _Engine(_lib.ARCH_BT4, num_layers, d_model, num_heads, d_ff, fp8=fp8, micro_batch=micro_batch, head_dtype=head_dtype,
                               act_dtype=act_dtype, stream_f32=stream_f32, norm_rms=norm_rms)
        self._engine.load(self._sd)

    @torch.no_grad()
    def forward(self, inp, compute_loss=False):
        """inp[0]: [b, seq_len, 8, 8, 19] -> policy [b, seq_len, 1929] (value.py:155-212). With compute_loss the
        reference's 6-tuple (value.py:197-202): inp[1] = policy targets [b, seq_len] (ignore_index 1928), inp[3] = value
        classes [b, seq_len, 1] (ignore_index 3) -> (policy, value logits [b, seq_len, 3], policy cross-entropy, value
        cross-entropy, targets, true_values). Forward values only: the losses carry no autograd graph."""
        x = inp[0]
        b, s = x.shape[0], x.shape[1]
        pol, wdl = self._engine.forward(x, want_wdl=compute_loss)
        policy = pol.view(b, s, VOCAB_RL)
        if not compute_loss:
            return policy
        targets, true_values = inp[1], inp[3]
        if true_values.shape[-1] != 1:
            # value.py:203-211 flattens a [b, 3] float target into F.cross_entropy's class-index slot, which torch rejects
            raise ValueError("value targets must be class indices of shape [..., 1] (the branch of value.py:200-202)")
        value_h = wdl.view(b, s, 3)
        loss_policy = cross_entropy(pol, targets.reshape(-1).to(pol.device), ignore_index=1928)
        loss_value = cross_entropy(wdl, true_values.reshape(-1).to(pol.device), ignore_index=3)
        return policy, value_h, loss_policy, loss_value, targets, true_values

    __call__ = forward

    @torch.no_grad()
    def get_move_from_fen_no_thinking(self, fen, T=1, device="cuda", force_legal=True, return_probs=False):
        planes = board.encode_fens([fen]).to(device)
        logits, _ = self._engine.forward(planes, want_wdl=False)
        mask = torch.from_numpy(board.legal_move_mask(fen)).to(device).unsqueeze(0) if force_legal else None
        idx, _ = self._sample(logits, mask, T)
        return policy_index[idx]

    @torch.no_grad()
    def get_batch_position_values(self, fens, device="cuda"):
        """[N,3] probabilities [black win, draw, white win] (value.py:275-317)."""
        if len(fens) == 0:
            return torch.empty(0, 3, device=device)
        planes = board.encode_fens(fens).to(device)
        _, wdl = self._engine.forward(planes)
        return torch.softmax(wdl, dim=-1)

    def get_position_value(self, fen, device="cuda"):
        return self.get_batch_position_values([fen], device)[0]

    def calculate_move_values(self, fen, device="cuda"):
        """(moves, value of each child for the side to move) (value.py:319-354)."""
        moves, fens = board.child_fens(fen)
        if not moves:
            return [], torch.empty(0, device=device)
        p = self.get_batch_position_values(fens, device)
        vals = 0.5 * p[:, 1] + (p[:, 2] if board.white_to_move(fen) else p[:, 0])
        return moves, vals

    @torch.no_grad()
    def get_best_move_value(self, fen, T=1, device="cuda", return_probs=False):
        moves, vals = self.calculate_move_values(fen, device)
        if not moves:
            raise ValueError("No legal moves available")
        if T == 0:
            best = int(torch.argmax(vals).item())
            probs = torch.zeros_like(vals)
            probs[best] = 1.0
        else:
            probs = torch.softmax(vals / T, dim=0)
            best = int(torch.multinomial(probs, num_samples=1).item())
        return (moves[best], probs.cpu().numpy()) if return_probs else moves[best]


class BT4Class(_ModelBase):
    """BT4-class encoder: post-LN with residual scaling, mish FFN, generated attention bias,
    attention policy gathered to the 1858 side-to-move-frame moves, WDL head."""

    def __init__(self, num_layers=15, d_model=1024, d_ff=1536, num_heads=32, fp8=False, micro_batch=0,
                 head_dtype=None, act_dtype="bf16", compress=32, hidden=256, gen=256, seed=0, stream_f32=None, ln_fold=None,
                 norm_rms=False, fp8_heads=None):
        """fp8_heads: with fp8, run policy_tokens_lin, queries_pol|keys_pol and value dense1 in e4m3 too (off by default)."""
        self.num_layers, self.d_model = num_layers, d_model
        self._shapes = bt4_shapes(num_layers, d_model, d_ff, num_heads, True, compress, hidden, gen)
        self._sd = _default_init(self._shapes, seed)
        self._engine = _Engine(_lib.ARCH_BT4CLASS, num_layers, d_model, num_heads, d_ff, fp8=fp8, micro_batch=micro_batch,
                               head_dtype=head_dtype, act_dtype=act_dtype, compress=compress, hidden=hidden, gen=gen,
                               stream_f32=stream_f32, ln_fold=ln_fold, norm_rms=norm_rms, fp8_lm_head=fp8_heads)
        self._engine.load(self._sd)

    @torch.no_grad()
    def forward(self, board_tokens):
        """board_tokens [B,8,8,19] -> (policy_logits [B,1858], wdl [B,3])."""
        return self._engine.forward(board_tokens)

    __call__ = forward

    @torch.no_grad()
    def get_move_from_fen_no_thinking(self, fen, T=1, device="cuda", force_legal=True, return_probs=False):
        planes = board.encode_fens([fen]).to(device)
        logits, _ = self._engine.forward(planes, want_wdl=False)
        mask = torch.from_numpy(board.legal_move_mask(fen, leela=True)).to(device).unsqueeze(0) if force_legal else None
        idx, probs = self._sample(logits, mask, T)
        move = policy_leela[idx]
        if not board.white_to_move(fen):
            move = move[0] + str(9 - int(move[1])) + move[2] + str(9 - int(move[3])) + move[4:]
        return (move, probs[0]) if return_probs else move
