"""Decode-step harness: the caller either side of the 4-bit linear in token generation.

A Llama-architecture decoder (RMSNorm, rotary GQA attention over a static KV cache, SwiGLU) whose
every ``nn.Linear`` is handed to ``BitsAndBytesLinearQuant4bit`` through ``jit``, and a greedy
decoding loop whose single-token step is captured in a HIP graph, the way the reference's
``CUDAGraphTransform`` replays a forward pass (thunder/transforms/cudagraph.py:47-226) over weights
tagged as static inputs (thunder/transforms/quantization.py:178,186).  Everything that is not a
linear (norms, rotary embedding, attention, sampling) is plain PyTorch by default: it is plumbing
around the path, not part of it.  With ``LlamaConfig.hip_glue`` the single-token step runs that work in
HIP kernels instead (``glue.py``: residual add + RMSNorm, rotary + cache update + attention,
SiLU * up; greedy sampling as a fourth), so that the step is bound by the 4-bit linears rather than by ~18 small
launches per layer.

``fused_projections=True`` builds Q/K/V and gate/up as ONE linear each ([6144, 4096] and
[28672, 4096] for Llama-3-8B).  NF4 blocks are 64 consecutive elements of a row, so the packed
weight of the row-concatenated matrix is the concatenation of the packed weights: fusing changes
no value, only the number of launches and the size of each weight stream.
"""

from __future__ import annotations

import time
from dataclasses import dataclass

import torch
import torch.nn.functional as F
from torch import nn


@dataclass
class LlamaConfig:
    n_layer: int = 32
    d_model: int = 4096
    n_head: int = 32
    n_kv_head: int = 8
    d_ff: int = 14336
    vocab: int = 128256
    rope_theta: float = 500000.0
    norm_eps: float = 1e-5
    max_seq: int = 640
    fused_projections: bool = False
    hip_glue: bool = False
    # with fused_projections: rows 2j / 2j+1 of the gate-up weight are row j of the gate / of the up projection (instead
    # of gate rows first, up rows after), so that the thread finishing a pair of outputs can apply SiLU(gate) * up itself
    gate_up_interleaved: bool = False
    # with hip_glue: let the 4-bit decode kernels' epilogues do the residual add, RMSNorm and SiLU * up where they can
    linear_epilogues: bool = True

    @property
    def head_dim(self) -> int:
        return self.d_model // self.n_head

    @classmethod
    def llama3_8b(cls, **kw) -> "LlamaConfig":
        return cls(**kw)

    @classmethod
    def tiny(cls, **kw) -> "LlamaConfig":
        base = dict(n_layer=2, d_model=512, n_head=8, n_kv_head=2, d_ff=1024, vocab=1024, max_seq=64)
        base.update(kw)
        return cls(**base)


def _rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    # x [B, T, heads, hd]; cos/sin [T, 1, hd] in x's dtype (each half repeated): x * cos + rotate_half(x) * sin
    x1, x2 = x.chunk(2, dim=-1)
    return torch.addcmul(x * cos, torch.cat((-x2, x1), dim=-1), sin)


class Attention(nn.Module):
    def __init__(self, cfg: LlamaConfig):
        super().__init__()
        self.cfg = cfg
        hd = cfg.head_dim
        if cfg.fused_projections:
            self.qkv_proj = nn.Linear(cfg.d_model, (cfg.n_head + 2 * cfg.n_kv_head) * hd, bias=False)
        else:
            self.q_proj = nn.Linear(cfg.d_model, cfg.n_head * hd, bias=False)
            self.k_proj = nn.Linear(cfg.d_model, cfg.n_kv_head * hd, bias=False)
            self.v_proj = nn.Linear(cfg.d_model, cfg.n_kv_head * hd, bias=False)
        self.o_proj = nn.Linear(cfg.n_head * hd, cfg.d_model, bias=False)

    def forward(self, x, pos, cos, sin, bias, kcache, vcache):
        cfg = self.cfg
        B, T, _ = x.shape
        hd, H, Hkv = cfg.head_dim, cfg.n_head, cfg.n_kv_head
        rep = H // Hkv
        if cfg.fused_projections:
            qkv = self.qkv_proj(x)
            qk, v = qkv[..., : (H + Hkv) * hd], qkv[..., (H + Hkv) * hd:]
        else:
            qk = torch.cat((self.q_proj(x), self.k_proj(x)), dim=-1)
            v = self.v_proj(x)
        qk = _rope(qk.reshape(B, T, H + Hkv, hd), cos, sin)  # q and k heads rotated in one go
        kcache.index_copy_(2, pos, qk[:, :, H:].transpose(1, 2))
        vcache.index_copy_(2, pos, v.reshape(B, T, Hkv, hd).transpose(1, 2))
        # grouped-query attention without expanding the cache: the `rep` query heads that share a
        # kv head become extra query rows of that head, row index r * T + t
        q = qk[:, :, :H].reshape(B, T, Hkv, rep, hd).permute(0, 2, 3, 1, 4).reshape(B, Hkv, rep * T, hd)
        if T == 1:
            # one query per head: two small batched matmuls beat a general attention kernel; the first
            # one also applies the scale and the additive mask (0 / -inf)
            scores = torch.baddbmm(bias.expand(B * Hkv, rep, -1), q.reshape(B * Hkv, rep, hd),
                                   kcache.reshape(B * Hkv, -1, hd).transpose(1, 2), alpha=hd ** -0.5)
            probs = torch.softmax(scores, dim=-1, dtype=torch.float32).to(q.dtype)
            y = torch.bmm(probs, vcache.reshape(B * Hkv, -1, hd)).reshape(B, Hkv, rep, hd)
        else:
            y = F.scaled_dot_product_attention(q, kcache, vcache, attn_mask=bias.repeat(rep, 1))
        y = y.reshape(B, Hkv, rep, T, hd).permute(0, 3, 1, 2, 4).reshape(B, T, H * hd)
        return self.o_proj(y)


class MLP(nn.Module):
    def __init__(self, cfg: LlamaConfig):
        super().__init__()
        self.cfg = cfg
        if cfg.fused_projections:
            self.gate_up_proj = nn.Linear(cfg.d_model, 2 * cfg.d_ff, bias=False)
        else:
            self.gate_proj = nn.Linear(cfg.d_model, cfg.d_ff, bias=False)
            self.up_proj = nn.Linear(cfg.d_model, cfg.d_ff, bias=False)
        self.down_proj = nn.Linear(cfg.d_ff, cfg.d_model, bias=False)

    def forward(self, x):
        if self.cfg.fused_projections and self.cfg.gate_up_interleaved:
            gu = self.gate_up_proj(x)
            gate, up = gu[..., 0::2], gu[..., 1::2]
        elif self.cfg.fused_projections:
            gate, up = self.gate_up_proj(x).chunk(2, dim=-1)
        else:
            gate, up = self.gate_proj(x), self.up_proj(x)
        return self.down_proj(F.silu(gate) * up)


class Block(nn.Module):
    def __init__(self, cfg: LlamaConfig):
        super().__init__()
        self.norm_1 = nn.RMSNorm(cfg.d_model, eps=cfg.norm_eps)
        self.attn = Attention(cfg)
        self.norm_2 = nn.RMSNorm(cfg.d_model, eps=cfg.norm_eps)
        self.mlp = MLP(cfg)

    def forward(self, x, pos, cos, sin, bias, kcache, vcache):
        x = x + self.attn(self.norm_1(x), pos, cos, sin, bias, kcache, vcache)
        return x + self.mlp(self.norm_2(x))


class Llama(nn.Module):
    """``forward(idx [B, T], pos [T], kcache, vcache) -> logits [B, vocab]`` of the LAST position.
    ``kcache`` / ``vcache``: [n_layer, B, n_kv_head, max_seq, head_dim], updated in place at ``pos``."""

    def __init__(self, cfg: LlamaConfig):
        super().__init__()
        self.cfg = cfg
        self.wte = nn.Embedding(cfg.vocab, cfg.d_model)
        self.blocks = nn.ModuleList(Block(cfg) for _ in range(cfg.n_layer))
        self.norm_f = nn.RMSNorm(cfg.d_model, eps=cfg.norm_eps)
        self.lm_head = nn.Linear(cfg.d_model, cfg.vocab, bias=False)
        inv = 1.0 / (cfg.rope_theta ** (torch.arange(0, cfg.head_dim, 2, dtype=torch.float32) / cfg.head_dim))
        ang = torch.outer(torch.arange(cfg.max_seq, dtype=torch.float32), inv).repeat(1, 2)
        self.register_buffer("rope_cos", ang.cos(), persistent=False)
        self.register_buffer("rope_sin", ang.sin(), persistent=False)
        self.register_buffer("key_index", torch.arange(cfg.max_seq), persistent=False)

    def _decode_step_glue(self, idx, pos, kcache, vcache):
        """The single-token forward with the HIP glue kernels: per layer four linears and four other
        launches.  The residual stream x is updated in place by add_rmsnorm, which also returns the
        normalised input of the next linear; `delta` is the branch output not yet added."""
        from . import glue

        cfg = self.cfg
        H, Hkv, eps = cfg.n_head, cfg.n_kv_head, cfg.norm_eps
        x = self.wte(idx)[:, 0, :].contiguous()
        if cfg.linear_epilogues and cfg.fused_projections and cfg.gate_up_interleaved and x.shape[0] <= 16:
            out = self._decode_step_epilogues(x, pos, kcache, vcache)
            if out is not None:
                return out
        delta = None
        for i, blk in enumerate(self.blocks):
            h = glue.add_rmsnorm(x, delta, blk.norm_1.weight, eps)
            a = blk.attn
            if cfg.fused_projections:
                qkv = a.qkv_proj(h)
            else:
                qkv = torch.cat((a.q_proj(h), a.k_proj(h), a.v_proj(h)), dim=-1)
            y = glue.attention_decode(qkv, pos, self.rope_cos, self.rope_sin, kcache[i], vcache[i], H, Hkv)
            delta = a.o_proj(y)
            h = glue.add_rmsnorm(x, delta, blk.norm_2.weight, eps)
            m = blk.mlp
            gate_up = m.gate_up_proj(h) if cfg.fused_projections else torch.cat((m.gate_proj(h), m.up_proj(h)), dim=-1)
            delta = m.down_proj(glue.silu_mul(gate_up, pairs=cfg.fused_projections and cfg.gate_up_interleaved))
        return self.lm_head(glue.add_rmsnorm(x, delta, self.norm_f.weight, eps))

    def _decode_step_epilogues(self, x, pos, kcache, vcache):
        """The single-token forward with the neighbours of every linear done in that linear's epilogue
        (``hip_matmul_nf4_epilogue``): the output and down projections add the residual, write the next norm's
        input times its weight and leave partial sums of squares; the QKV, gate-up and lm_head projections scale their
        sums by the 1 / rms those give, and the gate-up projection applies SiLU(gate) * up to its pairs of outputs.
        Per layer four linears and the attention kernel.  Returns None (before anything is launched) unless every
        linear runs as the 4-bit operator with fp32 absmax at a shape the kernels take."""
        from . import glue
        from .transforms import quantization as Q

        cfg = self.cfg
        H, Hkv, eps = cfg.n_head, cfg.n_kv_head, cfg.norm_eps
        lins = [l for blk in self.blocks for l in (blk.attn.qkv_proj, blk.attn.o_proj, blk.mlp.gate_up_proj, blk.mlp.down_proj)]
        # The library's verdict and the operator arguments of every linear depend on (rows of x, device, what the
        # compiled module planned for each weight) only: asked once and kept on the model, so that an eager step does not
        # repeat a few hundred host-side queries per token.  The plan objects are part of the key (and kept alive by it):
        # a module that is re-planned -- its override tables changed -- gets a fresh answer.
        plans = tuple(getattr(l.weight, "_planned_operator", None) for l in lins + [self.lm_head])
        key = (x.shape[0], x.device, tuple(id(p) for p in plans))
        cached = self.__dict__.get("_epilogue_chain")
        if cached is None or cached[0] != key:
            served = _chain_served(x.shape[0], self)
            cached = (key, plans, served, {id(l): _planned_nf4(l) for l in lins + [self.lm_head]} if served else None)
            self.__dict__["_epilogue_chain"] = cached
        if not cached[2]:
            return None
        args = cached[3]
        ep = Q.hip_matmul_nf4_epilogue
        r = x
        xn = ss = None
        for i, blk in enumerate(self.blocks):
            a, m = blk.attn, blk.mlp
            if i == 0:
                qkv = a.qkv_proj(glue.add_rmsnorm(r, None, blk.norm_1.weight, eps))
            else:
                qkv = ep(xn, *args[id(a.qkv_proj)], rowscale=(ss, eps))
            y = glue.attention_decode(qkv, pos, self.rope_cos, self.rope_sin, kcache[i], vcache[i], H, Hkv)
            r, xn, ss = ep(y, *args[id(a.o_proj)], resid_norm=(r, blk.norm_2.weight))
            h = ep(xn, *args[id(m.gate_up_proj)], rowscale=(ss, eps), silu_pairs=True)
            nxt = self.blocks[i + 1].norm_1.weight if i + 1 < len(self.blocks) else self.norm_f.weight
            r, xn, ss = ep(h, *args[id(m.down_proj)], resid_norm=(r, nxt))
        return ep(xn, *args[id(self.lm_head)], rowscale=(ss, eps))

    def forward(self, idx, pos, kcache, vcache):
        if self.cfg.hip_glue and idx.shape[1] == 1 and idx.is_cuda and self.wte.weight.dtype == torch.bfloat16:
            return self._decode_step_glue(idx, pos, kcache, vcache)
        x = self.wte(idx)
        cos = self.rope_cos.index_select(0, pos)[:, None, :].to(x.dtype)
        sin = self.rope_sin.index_select(0, pos)[:, None, :].to(x.dtype)
        # additive attention mask [T, max_seq]: 0 where key s is visible to the query at pos[t], else -inf
        visible = self.key_index[None, :] <= pos[:, None]
        bias = torch.zeros(visible.shape, dtype=x.dtype, device=x.device).masked_fill(~visible, float("-inf"))
        for i, blk in enumerate(self.blocks):
            x = blk(x, pos, cos, sin, bias, kcache[i], vcache[i])
        return self.lm_head(self.norm_f(x[:, -1:, :])).squeeze(1)


def _planned_nf4(lin: nn.Linear):
    """``(qweight, bias, absmax, quant_map, blocksize, dtype, shape)`` when ``lin`` runs as the operator
    ``hip_matmul_nf4`` (4-bit weight, fp32 absmax) in the compiled module, else None."""
    planned = getattr(lin.weight, "_planned_operator", None)
    if planned is None or planned[0] != "hip_matmul_nf4":
        return None
    _, packed, rest = planned
    return (packed, lin.bias, *rest)


def _chain_served(rows: int, model: "Llama") -> bool:
    """Do the decode kernels take, at ``rows`` rows of x, every epilogue that ``Llama._decode_step_epilogues`` asks of
    the model's 4-bit linears?  (Asked before the step launches anything: a refusal half way would leave it nowhere.)"""
    from . import _lib, functional

    lib = _lib.load()

    def served(lin, producer=None, **kw):
        args = _planned_nf4(lin)
        if args is None:
            return False
        _, _, absmax, _, blocksize, dtype, shape = args
        if producer is not None:  # row scale: as many partial sums as the producing linear leaves
            kw["rowscale_parts"] = lib.nf4hip_gemv_norm_parts(rows, producer.out_features, producer.in_features)
            if kw["rowscale_parts"] <= 0:
                return False
        return functional.epilogue_served(rows, shape, blocksize, dtype, isinstance(absmax, functional.NestedAbsmax), **kw)

    for blk in model.blocks:
        a, m = blk.attn, blk.mlp
        if not (served(a.qkv_proj, m.down_proj) and served(a.o_proj, resid_norm=True)
                and served(m.gate_up_proj, a.o_proj, silu_pairs=True) and served(m.down_proj, resid_norm=True)):
            return False
    return served(model.lm_head, model.blocks[-1].mlp.down_proj)


def build_llama(cfg: LlamaConfig, device="cuda", dtype=torch.bfloat16, seed: int = 0) -> Llama:
    """Random-init weights ~ N(0, 0.02), drawn on ``device`` from one seeded generator."""
    with torch.device("meta"):
        model = Llama(cfg)
    model = model.to_empty(device=device)
    g = torch.Generator(device=device).manual_seed(seed)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if p.ndim == 1:
                p.data = torch.ones_like(p, dtype=dtype)
            else:
                w = torch.empty(p.shape, device=device, dtype=torch.float32).normal_(0.0, 0.02, generator=g)
                p.data = w.to(dtype)
                del w
        inv = 1.0 / (cfg.rope_theta ** (torch.arange(0, cfg.head_dim, 2, dtype=torch.float32, device=device) / cfg.head_dim))
        ang = torch.outer(torch.arange(cfg.max_seq, dtype=torch.float32, device=device), inv).repeat(1, 2)
        model.rope_cos, model.rope_sin = ang.cos(), ang.sin()
        model.key_index = torch.arange(cfg.max_seq, device=device)
    return model.eval().requires_grad_(False)


def new_caches(cfg: LlamaConfig, batch: int, device="cuda", dtype=torch.bfloat16):
    shape = (cfg.n_layer, batch, cfg.n_kv_head, cfg.max_seq, cfg.head_dim)
    return torch.zeros(shape, device=device, dtype=dtype), torch.zeros(shape, device=device, dtype=dtype)


@torch.no_grad()
def greedy_decode(model, cfg: LlamaConfig, prompt: torch.Tensor, n_new: int, use_graph: bool = True):
    """Greedy decoding of ``n_new`` tokens after ``prompt`` [B, P].  Returns ``(tokens [B, n_new],
    stats)`` with the prefill and decode wall times (GPU-synchronised).

    With ``use_graph`` one decode step -- forward, argmax, feeding the token and the position back
    into their static buffers -- is captured in a HIP graph and replayed; the host only enqueues
    replays and copies each step's token out, and synchronises once at the end.
    """
    B, P = prompt.shape
    dev = prompt.device
    assert P + n_new <= cfg.max_seq
    kcache, vcache = new_caches(cfg, B, dev, model.wte.weight.dtype)

    def sync():
        if dev.type == "cuda":
            torch.cuda.synchronize(dev)

    sync()
    t0 = time.perf_counter()
    logits = model(prompt, torch.arange(P, device=dev), kcache, vcache)
    first = logits.argmax(-1, keepdim=True)
    sync()
    t_prefill = time.perf_counter() - t0

    tok = first.clone()
    pos = torch.full((1,), P, device=dev, dtype=torch.long)
    out = torch.empty(n_new, B, device=dev, dtype=torch.long)
    out[0] = first[:, 0]

    def step():
        logits = model(tok, pos, kcache, vcache)
        if cfg.hip_glue and logits.is_cuda and logits.dtype == torch.bfloat16:
            from . import glue

            glue.argmax_into(logits, tok.view(-1), pos)  # the next token and pos += 1 in one launch
            return
        tok.copy_(logits.argmax(-1, keepdim=True))
        pos.add_(1)

    graph = None
    if use_graph and n_new > 1 and dev.type == "cuda":
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            step()  # allocations, workspaces of this stream, lazy library state
            step()
            tok.copy_(first)  # roll the state back: the steps above wrote cache rows P, P+1, which
            pos.fill_(P)      # the real steps rewrite before reading them
            torch.cuda.synchronize(dev)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                step()
            tok.copy_(first)  # capture does not execute, but keep the state explicit
            pos.fill_(P)
        torch.cuda.current_stream(dev).wait_stream(side)

    sync()
    t1 = time.perf_counter()
    for i in range(1, n_new):
        if graph is not None:
            graph.replay()
        else:
            step()
        out[i] = tok[:, 0]
    sync()
    t_decode = time.perf_counter() - t1
    stats = {
        "prefill_s": t_prefill,
        "decode_s": t_decode,
        "decode_steps": n_new - 1,
        "decode_tok_per_s": B * (n_new - 1) / t_decode if n_new > 1 else 0.0,
        "graph": graph is not None,
    }
    return out.t().contiguous(), stats


def fuse_state_dict(sd: dict, cfg: LlamaConfig) -> dict:
    """State dict of the ``fused_projections=True`` model from that of the unfused one: Q/K/V and
    gate/up weights concatenated along the output dimension."""
    out = {}
    for k, v in sd.items():
        if k.endswith(("k_proj.weight", "v_proj.weight", "up_proj.weight")) and "gate_up" not in k:
            continue
        if k.endswith("q_proj.weight"):
            base = k[: -len("q_proj.weight")]
            out[base + "qkv_proj.weight"] = torch.cat([v, sd[base + "k_proj.weight"], sd[base + "v_proj.weight"]], dim=0)
        elif k.endswith("gate_proj.weight"):
            base = k[: -len("gate_proj.weight")]
            up = sd[base + "up_proj.weight"]
            if cfg.gate_up_interleaved:  # rows 2j / 2j+1 = gate row j / up row j
                out[base + "gate_up_proj.weight"] = torch.stack([v, up], dim=1).reshape(2 * v.shape[0], v.shape[1])
            else:
                out[base + "gate_up_proj.weight"] = torch.cat([v, up], dim=0)
        else:
            out[k] = v
    return out
