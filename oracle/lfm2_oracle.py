"""CPU oracle for the LFM2 decode/prefill path.  TEST INFRASTRUCTURE ONLY.

This file restates, in plain CPU PyTorch, the algorithms of the reference
engine so that the HIP path can be checked against it.  It is never imported by
the product package: only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may use it, and only as the checker.

Reference files followed (paths under the reference checkout,
``src/climbing_gym/inference`` unless noted):

* eager engine .............. ``lfm25_engine.py`` (prefill 605-684, 1014-1106;
  decode 1223-1362, 1424-1449, 1533-1572; sampling 1574-1617, 1759-1790)
* fused decode step ......... ``lfm25_cuda.py:128-192``
* rounding of fused kernels . ``lfm25_cuda_kernels.py:32-151``
* e4m3 quantisation / GEMM .. ``lfm25_fp8.py:17-105``
* e4m3 KV store / decode .... ``lfm25_fp8_kv.py:28-167``
* sampler bookkeeping ....... ``lfm25_sampling.py:9-58``, ``lfm25_session.py:34-56``
* stop automaton ............ ``text_stops.py:17-45``
* config schema ............. ``models/lfm2.py:176-260``

How each part is pinned (see ``tests/test_oracle_*.py``):

* full prefill + cached decode: against ``transformers.Lfm2ForCausalLM``
  (an independent implementation) at 1e-5 in fp32, plus cached == recompute,
  padded-chunk == per-prompt.
* RMSNorm / RoPE: against the Transformers routines (RoPE bitwise in bf16).
* short conv: brute force from the definition of a causal depthwise conv.
* e4m3 rounding: brute-force nearest-code search over all 256 codes.
* top-k / top-p filter: brute-force Python loops on tiny vocabularies.
* stop automaton, chunk planner, capacity rounding: known answers held by the
  reference's own tests.

Parity unpinned (nothing but the text of the reference fixes them): the exact
token drawn at temperature > 0 (``torch.multinomial`` with a CPU generator on the
reference CPU engine, Triton's ``tl.rand`` stream on its GPU path).  Only the
distribution is checked for those.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Mapping, Sequence

import torch
import torch.nn.functional as F

E4M3_MAX = 448.0
LOG2E = 1.4426950408889634


# --------------------------------------------------------------------------- config
@dataclass
class OracleConfig:
    """Subset of ``models/lfm2.py:176-227`` that the inference path reads."""

    vocab_size: int = 65536
    hidden_size: int = 2048
    mlp_hidden_size: int = 8192
    num_hidden_layers: int = 16
    num_attention_heads: int = 32
    num_key_value_heads: int = 8
    max_position_embeddings: int = 128000
    rope_theta: float = 1_000_000.0
    norm_eps: float = 1e-5
    conv_kernel_size: int = 3
    layer_types: tuple = ()
    eos_token_id: int = 7

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads


# --------------------------------------------------------------------------- primitives
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``lfm25_engine.py:1741-1746``: fp32 statistics, cast, then scale."""
    dt = x.dtype
    h = x.float()
    h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + eps)
    return (h.to(dt) * weight).to(dt)


def apply_rotary(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Rotate-half with coefficients in the activation dtype (``lfm25_engine.py:1749-1756``)."""
    half = x.shape[-1] // 2
    a, b = x[..., :half], x[..., half:]
    c, s = cos.to(x.dtype), sin.to(x.dtype)
    return torch.cat((a * c - b * s, b * c + a * s), -1).to(x.dtype)


def rope_tables(head_dim: int, theta: float, length: int):
    """fp32 cos/sin ``[length, head_dim/2]`` (``lfm25_engine.py:1004-1012``)."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    ang = torch.arange(length, dtype=torch.float32)[:, None] * inv[None, :]
    return ang.cos(), ang.sin()


def top_k_top_p_filter(logits: torch.Tensor, top_k: int, top_p: float) -> torch.Tensor:
    """``lfm25_engine.py:1759-1774``: ties with the k-th value are kept; the
    nucleus drops every sorted rank whose cumulative mass exceeds ``top_p``
    except rank 0 (no shift)."""
    out = logits
    if 0 < top_k < logits.size(-1):
        kth = torch.topk(out, top_k, dim=-1).values[:, -1:]
        out = out.masked_fill(out < kth, -math.inf)
    if top_p < 1.0:
        vals, idx = torch.sort(out, descending=True, dim=-1)
        drop = torch.softmax(vals, -1).cumsum(-1) > top_p
        drop[:, 0] = False
        vals = vals.masked_fill(drop, -math.inf)
        out = torch.full_like(out, -math.inf).scatter(1, idx, vals)
    return out


def sampling_logprobs(logits: torch.Tensor, tokens: torch.Tensor, temperature: float, top_k: int, top_p: float):
    """Third result of ``_sample`` (``lfm25_engine.py:1591-1608``): log-probability of ``tokens`` under the
    distribution they were drawn from, softmax of the tempered logits with everything outside the top-k / nucleus
    support at -inf; at temperature 0 it is the raw log-softmax (``:1594-1596``).  A token outside the support gets
    -inf."""
    lf = logits.float()
    if temperature == 0.0:
        return lf.gather(1, tokens[:, None])[:, 0] - torch.logsumexp(lf, -1)
    kept = top_k_top_p_filter(lf / float(temperature), top_k, top_p)
    return kept.gather(1, tokens[:, None])[:, 0] - torch.logsumexp(kept, -1)


def repetition_penalty(logits, seen, penalty):
    """``lfm25_engine.py:1777-1790``."""
    if seen is None or penalty == 1.0:
        return logits
    return torch.where(seen, torch.where(logits < 0, logits * penalty, logits / penalty), logits)


def greedy_with_logprob(logits: torch.Tensor):
    """argmax (first index on ties) and raw log-softmax of the pick (``lfm25_engine.py:1591-1597``)."""
    lf = logits.float()
    tok = lf.argmax(-1)
    # the normaliser in float64: an fp32 running sum drops terms below half an ulp of a dominant one
    return tok, (lf.double().gather(1, tok[:, None])[:, 0] - torch.logsumexp(lf.double(), -1)).float()


# --------------------------------------------------------------------------- weights
@dataclass
class OracleLayer:
    kind: str
    operator_norm: torch.Tensor
    ffn_norm: torch.Tensor
    w13: torch.Tensor
    w2: torch.Tensor
    cache_index: int
    qkv: torch.Tensor | None = None
    out: torch.Tensor | None = None
    q_norm: torch.Tensor | None = None
    k_norm: torch.Tensor | None = None
    conv_in: torch.Tensor | None = None
    conv_w: torch.Tensor | None = None
    conv_out: torch.Tensor | None = None


def _get(state: Mapping[str, torch.Tensor], key: str) -> torch.Tensor:
    """Optional ``model.`` prefix (``lfm25_engine.py:1700-1710``)."""
    for k in (key, key[6:] if key.startswith("model.") else "model." + key):
        if k in state:
            return state[k]
    raise KeyError(key)


def _has(state, key):
    return key in state or (key[6:] if key.startswith("model.") else "model." + key) in state


def pack_layers(cfg: OracleConfig, state, dtype):
    """``lfm25_engine.py:134-223``: w13=[w1;w3], qkv=[q;k;v], conv weight [H,1,3]->[H,3]."""
    t = lambda k: _get(state, k).detach().to(dtype).contiguous()
    layers, na, nc = [], 0, 0
    for i, kind in enumerate(cfg.layer_types):
        p = f"model.layers.{i}"
        common = dict(operator_norm=t(f"{p}.operator_norm.weight"), ffn_norm=t(f"{p}.ffn_norm.weight"),
                      w13=torch.cat([t(f"{p}.feed_forward.w1.weight"), t(f"{p}.feed_forward.w3.weight")]).contiguous(),
                      w2=t(f"{p}.feed_forward.w2.weight"))
        if kind == "full_attention":
            layers.append(OracleLayer("attn", cache_index=na, **common,
                                      qkv=torch.cat([t(f"{p}.self_attn.{n}_proj.weight") for n in "qkv"]).contiguous(),
                                      out=t(f"{p}.self_attn.out_proj.weight"),
                                      q_norm=t(f"{p}.self_attn.q_layernorm.weight"),
                                      k_norm=t(f"{p}.self_attn.k_layernorm.weight")))
            na += 1
        elif kind == "conv":
            layers.append(OracleLayer("conv", cache_index=nc, **common,
                                      conv_in=t(f"{p}.conv.in_proj.weight"),
                                      conv_w=t(f"{p}.conv.conv.weight")[:, 0, :].contiguous(),
                                      conv_out=t(f"{p}.conv.out_proj.weight")))
            nc += 1
        else:
            raise ValueError(kind)
    embed = t("model.embed_tokens.weight")
    head = t("model.lm_head.weight") if _has(state, "model.lm_head.weight") else embed
    return embed, t("model.embedding_norm.weight"), head, layers, na, nc


@dataclass
class OracleCache:
    """Dense slot cache of ``lfm25_engine.py:370-431``: k/v ``[La, slots, cap, KH, D]``,
    conv state ``[Lc, slots, H, 3]`` (index 2 = newest tap), ``seq_lens [slots]``."""

    k: torch.Tensor
    v: torch.Tensor
    conv: torch.Tensor
    seq_lens: torch.Tensor

    def rows(self, a, b):
        return OracleCache(self.k[:, a:b], self.v[:, a:b], self.conv[:, a:b], self.seq_lens[a:b])


def plan_prefill_chunks(lengths: Sequence[int], budget: int):
    """Greedy contiguous grouping of ``lfm25_engine.py:646-665``: extend while
    ``(n+1)*max_len <= budget``; the first prompt of a chunk is always taken."""
    chunks, start, n = [], 0, len(lengths)
    while start < n:
        end, width = start, 0
        while end < n:
            cand = max(width, lengths[end])
            if end > start and (end - start + 1) * cand > budget:
                break
            width, end = cand, end + 1
        chunks.append((start, end, width))
        start = end
    return chunks


def graph_capacity(cache_len: int, batch: int, max_model_len: int) -> int:
    """``lfm25_cuda.py:216-217``."""
    a = 32 if batch >= 64 else 128
    return min(max_model_len, (cache_len + a - 1) // a * a)


# --------------------------------------------------------------------------- eager engine
class OracleEngine:
    """CPU restatement of ``LFM25Engine`` (eager path)."""

    def __init__(self, cfg: OracleConfig, state, dtype=torch.float32, max_model_len: int | None = None, fp8=()):
        """``fp8`` names the parts that emulate W8A8 / e4m3-KV arithmetic: any of "mlp", "head", "operators", "kv"
        (``lfm25_cuda.py:97-106,172-176``; "operators" is the QKV/out and conv in/out extension).  Emulation means
        quantise-dequantise with the rules of ``k_quantize_rows`` / ``k_store_kv`` around an exact matmul."""
        self.cfg, self.dtype, self.fp8 = cfg, dtype, frozenset(fp8)
        (self.embed, self.final_norm, self.head, self.layers,
         self.n_attn, self.n_conv) = pack_layers(cfg, state, dtype)
        self.max_model_len = int(max_model_len or min(cfg.max_position_embeddings, 32768))
        self.QH, self.KH, self.D = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
        self.scale = self.D ** -0.5
        self.cos, self.sin = rope_tables(self.D, cfg.rope_theta, self.max_model_len)
        # tests may set this to a list: every layer's input hidden state is then appended as
        # ("prefill" | "decode", layer index, tensor) -- the `return_hidden` idea of lfm25_engine.py:1097-1098 per layer
        self.hidden_trace = None

    # ---- cache
    def empty_cache(self, slots: int, cap: int) -> OracleCache:
        z = lambda *s: torch.zeros(s, dtype=self.dtype)
        return OracleCache(z(self.n_attn, slots, cap, self.KH, self.D), z(self.n_attn, slots, cap, self.KH, self.D),
                           z(self.n_conv, slots, self.cfg.hidden_size, 3), torch.zeros(slots, dtype=torch.int32))

    # ---- shared pieces
    def _lin(self, x, w, part):
        """``F.linear``, or its W8A8 emulation when ``part`` is switched to FP8."""
        if part not in self.fp8:
            return F.linear(x, w)
        xq, xs = k_quantize_rows(x.reshape(-1, x.shape[-1]))
        wq, ws = k_quantize_rows(w)
        return k_fp8_linear(xq, xs, wq, ws, x.dtype).reshape(*x.shape[:-1], w.shape[0])

    def _kv(self, k, v):
        """What a later decode step reads back from the cache: the tensors themselves, or their e4m3 round trip."""
        if "kv" not in self.fp8:
            return k, v
        kq, ks, vq, vs = k_store_kv(k, v)
        return (kq.float() * ks[..., None]).to(k.dtype), (vq.float() * vs[..., None]).to(v.dtype)

    def _mlp(self, layer, x):
        # bf16 runs w1 and w3 separately, fp32 fused (lfm25_engine.py:1300-1304).
        I = layer.w13.size(0) // 2
        if x.dtype == torch.bfloat16 and "mlp" not in self.fp8:
            g, u = F.linear(x, layer.w13[:I]), F.linear(x, layer.w13[I:])
        else:
            g, u = self._lin(x, layer.w13, "mlp").chunk(2, -1)
        return self._lin(F.silu(g) * u, layer.w2, "mlp")

    def _qkv_split(self, layer, x, fused_ok: bool):
        H, kvw = self.cfg.hidden_size, self.KH * self.D
        if "operators" in self.fp8 or (fused_ok and x.dtype != torch.bfloat16):
            y = self._lin(x, layer.qkv, "operators")
            q, k, v = y[..., :H], y[..., H:H + kvw], y[..., H + kvw:]
        else:  # three projections (lfm25_engine.py:1318-1321, 1377-1379)
            q, k, v = (F.linear(x, w) for w in layer.qkv.split((H, kvw, kvw)))
        return q, k, v

    # ---- padded-chunk prefill (lfm25_engine.py:1050-1106, 1396-1422, 1478-1511)
    def prefill_padded(self, cache: OracleCache, ids: torch.Tensor, lengths: torch.Tensor | None = None):
        B, T = ids.shape
        pos = torch.arange(T)
        cos, sin = self.cos[pos].view(1, T, 1, -1), self.sin[pos].view(1, T, 1, -1)
        h = F.embedding(ids, self.embed)
        for index, L in enumerate(self.layers):
            if self.hidden_trace is not None:
                self.hidden_trace.append(("prefill", index, h.clone()))
            x = rms_norm(h, L.operator_norm, self.cfg.norm_eps)
            if L.kind == "attn":
                q, k, v = self._qkv_split(L, x, fused_ok=False)
                q = rms_norm(q.reshape(B, T, self.QH, self.D), L.q_norm, self.cfg.norm_eps)
                k = rms_norm(k.reshape(B, T, self.KH, self.D), L.k_norm, self.cfg.norm_eps)
                v = v.reshape(B, T, self.KH, self.D)
                q, k = apply_rotary(q, cos, sin), apply_rotary(k, cos, sin)
                cache.k[L.cache_index, :B, :T], cache.v[L.cache_index, :B, :T] = self._kv(k, v)
                g = self.QH // self.KH
                o = F.scaled_dot_product_attention(q.transpose(1, 2), k.repeat_interleave(g, 2).transpose(1, 2),
                                                   v.repeat_interleave(g, 2).transpose(1, 2), is_causal=True)
                y = self._lin(o.transpose(1, 2).reshape(B, T, -1), L.out, "operators")
            else:
                b, c, xp = self._lin(x, L.conv_in, "operators").chunk(3, -1)
                bx = b * xp
                conv = F.conv1d(bx.transpose(1, 2), L.conv_w.unsqueeze(1), padding=2,
                                groups=self.cfg.hidden_size)[..., :T].transpose(1, 2)
                st = cache.conv[L.cache_index, :B]
                st.zero_()
                ln = lengths if lengths is not None else torch.full((B,), T)
                idx = ln[:, None].long() + torch.arange(-3, 0)[None, :]
                hist = bx.gather(1, idx.clamp_min(0)[:, :, None].expand(-1, -1, bx.size(-1)))
                st.copy_(torch.where(idx[:, :, None] >= 0, hist, torch.zeros((), dtype=hist.dtype)).transpose(1, 2))
                y = self._lin(c * conv, L.conv_out, "operators")
            h = h + y
            h = h + self._mlp(L, rms_norm(h, L.ffn_norm, self.cfg.norm_eps))
        if lengths is None:
            cache.seq_lens[:B] = T
            last = h[:, -1]
        else:
            cache.seq_lens[:B] = lengths.to(torch.int32)
            last = h[torch.arange(B), lengths.long() - 1]
        return self._lin(rms_norm(last, self.final_norm, self.cfg.norm_eps), self.head, "head")

    def prefill(self, prompts: Sequence[Sequence[int]], cache: OracleCache | None = None,
                cap: int | None = None, max_prefill_tokens: int | None = None):
        """``lfm25_engine.py:605-684``: per-prompt when unbudgeted, otherwise padded
        chunks from :func:`plan_prefill_chunks` (right-padded with token 0)."""
        lens = [len(p) for p in prompts]
        if cache is None:
            cache = self.empty_cache(len(prompts), cap or max(lens))
        logits = torch.empty(len(prompts), self.cfg.vocab_size, dtype=self.dtype)
        if max_prefill_tokens is None:
            for i, p in enumerate(prompts):
                logits[i] = self.prefill_padded(cache.rows(i, i + 1), torch.tensor([list(p)]))[0]
        else:
            for a, b, width in plan_prefill_chunks(lens, max_prefill_tokens):
                ids = torch.zeros(b - a, width, dtype=torch.long)
                for r, p in enumerate(prompts[a:b]):
                    ids[r, :len(p)] = torch.tensor(list(p))
                logits[a:b] = self.prefill_padded(cache.rows(a, b), ids, torch.tensor(lens[a:b]))
        return cache, logits

    # ---- one decode token per slot (lfm25_engine.py:1223-1278, 1306-1362, 1424-1449, 1533-1572)
    def append_tokens(self, cache: OracleCache, slots: torch.Tensor, tokens: torch.Tensor):
        slots = slots.long()
        pos = cache.seq_lens[slots].long()
        if (pos >= cache.k.size(2)).any():
            raise RuntimeError("cache capacity exceeded")
        n = slots.numel()
        cos, sin = self.cos[pos].unsqueeze(1), self.sin[pos].unsqueeze(1)
        h = F.embedding(tokens.long(), self.embed)
        for index, L in enumerate(self.layers):
            if self.hidden_trace is not None:
                self.hidden_trace.append(("decode", index, h.clone()))
            x = rms_norm(h, L.operator_norm, self.cfg.norm_eps)
            if L.kind == "attn":
                q, k, v = self._qkv_split(L, x, fused_ok=True)
                q = rms_norm(q.reshape(n, self.QH, self.D), L.q_norm, self.cfg.norm_eps)
                k = rms_norm(k.reshape(n, self.KH, self.D), L.k_norm, self.cfg.norm_eps)
                q, k = apply_rotary(q, cos, sin), apply_rotary(k, cos, sin)
                kc, vc = cache.k[L.cache_index], cache.v[L.cache_index]
                kc[slots, pos], vc[slots, pos] = self._kv(k, v.reshape(n, self.KH, self.D))
                g = self.QH // self.KH
                outs = []
                for r in range(n):  # per-row form, lfm25_engine.py:1562-1572
                    t = int(pos[r]) + 1
                    kh = kc[slots[r], :t].repeat_interleave(g, 1).permute(1, 0, 2)
                    vh = vc[slots[r], :t].repeat_interleave(g, 1).permute(1, 0, 2)
                    s = torch.einsum("hd,htd->ht", q[r], kh) * self.scale
                    p = torch.softmax(s, -1, dtype=torch.float32).to(q.dtype)
                    outs.append(torch.einsum("ht,htd->hd", p, vh).reshape(-1))
                y = self._lin(torch.stack(outs), L.out, "operators")
            else:
                b, c, xp = self._lin(x, L.conv_in, "operators").chunk(3, -1)
                bx = b * xp
                st = cache.conv[L.cache_index]
                new = torch.roll(st[slots], -1, -1)
                new[:, :, -1] = bx
                st[slots] = new
                y = self._lin(c * (new * L.conv_w[None]).sum(-1), L.conv_out, "operators")
            h = h + y
            h = h + self._mlp(L, rms_norm(h, L.ffn_norm, self.cfg.norm_eps))
        cache.seq_lens[slots] += 1
        if self.hidden_trace is not None:
            self.hidden_trace.append(("decode", len(self.layers), h.clone()))
        return self._lin(rms_norm(h, self.final_norm, self.cfg.norm_eps), self.head, "head")

    # ---- sampling (lfm25_engine.py:1574-1609)
    def sample(self, logits, *, temperature=0.0, top_k=0, top_p=1.0, generator=None, seen=None, penalty=1.0):
        """``lfm25_engine.py:1574-1609``: (token, raw log-probability)."""
        tok, raw, _ = OracleEngine.sample_with_sampling_logprobs(self, logits, temperature=temperature, top_k=top_k, top_p=top_p,
                                                         generator=generator, seen=seen, penalty=penalty)
        return tok, raw

    def sample_with_sampling_logprobs(self, logits, *, temperature=0.0, top_k=0, top_p=1.0, generator=None, seen=None,
                                      penalty=1.0):
        """``lfm25_engine.py:1574-1609`` with all three results: the token, its log-probability under softmax of the
        (penalised) logits, and under the distribution it was drawn from (``sampling_logprobs`` below)."""
        lf = repetition_penalty(logits.float(), seen, penalty)
        if temperature == 0.0:
            tok = lf.argmax(-1)
        else:
            probs = torch.softmax(top_k_top_p_filter(lf / temperature, top_k, top_p), -1)
            tok = torch.multinomial(probs, 1, generator=generator)[:, 0]
        raw = lf.gather(1, tok[:, None])[:, 0] - torch.logsumexp(lf, -1)
        return tok, raw, sampling_logprobs(lf, tok, temperature, top_k, top_p)

    def generate(self, prompts, max_new_tokens: int, *, temperature=0.0, top_k=0, top_p=1.0, seed=0,
                 max_prefill_tokens=None, return_logits=False):
        """Fixed-length generation (``ignore_eos`` form, ``lfm25_engine.py:867-931``);
        the first token comes from the prefill logits."""
        cap = max(len(p) for p in prompts) + max_new_tokens
        cache, logits = self.prefill(prompts, cap=cap, max_prefill_tokens=max_prefill_tokens)
        gen = torch.Generator().manual_seed(int(seed))
        B = len(prompts)
        toks = torch.empty(B, max_new_tokens, dtype=torch.long)
        lps = torch.empty(B, max_new_tokens)
        trace = []
        slots = torch.arange(B)
        for s in range(max_new_tokens):
            if return_logits:
                trace.append(logits.clone())
            t, lp = self.sample(logits, temperature=temperature, top_k=top_k, top_p=top_p, generator=gen)
            toks[:, s], lps[:, s] = t, lp
            if s + 1 < max_new_tokens:
                logits = self.append_tokens(cache, slots, t)
        return (toks, lps, trace) if return_logits else (toks, lps)


# --------------------------------------------------------------------------- fused-kernel rounding semantics
def _rt(x: torch.Tensor, dt) -> torch.Tensor:
    """Round an fp32 tensor to ``dt`` and come back to fp32."""
    return x.to(dt).float()


def k_rms_norm(x, weight, eps, residual=None):
    """``lfm25_cuda_kernels.py:32-55``: returns ``(out, summed)``; the sum and the
    normalised value are each rounded to the model dtype before the next step."""
    dt = x.dtype
    h = x.float()
    if residual is not None:
        h = _rt(h + residual.float(), dt)
    summed = h.to(dt) if residual is not None else x
    n = _rt(h * torch.rsqrt((h * h).sum(-1, keepdim=True) / h.size(-1) + eps), dt)
    return (n * weight.float()).to(dt), summed


def k_swiglu(x):
    """``lfm25_cuda_kernels.py:58-72``: silu rounded to dtype, then times ``up``."""
    dt = x.dtype
    g, u = x.float().chunk(2, -1)
    return (_rt(g / (1.0 + torch.exp(-g)), dt) * u).to(dt)


def k_conv_update(bcx, weight, state, active=None, slot_ids=None):
    """``lfm25_cuda_kernels.py:75-110``.  ``state`` ``[slots,H,3]`` is updated in place
    for active rows; products are rounded to dtype, summed in fp32, rounded again."""
    dt = bcx.dtype
    M = bcx.size(0)
    b, c, xp = bcx.float().chunk(3, -1)
    bx = _rt(b * xp, dt)
    slots = torch.arange(M) if slot_ids is None else slot_ids.long().clamp_min(0)
    st = state[slots].float()
    w = weight.float()
    conv = _rt(_rt(st[:, :, 1] * w[:, 0], dt) + _rt(st[:, :, 2] * w[:, 1], dt) + _rt(bx * w[:, 2], dt), dt)
    new = torch.stack((st[:, :, 1], st[:, :, 2], bx), -1).to(dt)
    on = torch.ones(M, dtype=torch.bool) if active is None else active.bool()
    for r in range(M):
        if on[r]:
            state[slots[r]] = new[r]
    return (c * conv).to(dt)


def k_prepare_qkv(x, q_w, k_w, cos, sin, positions, QH, KH, D, eps):
    """``lfm25_cuda_kernels.py:113-151``: per-head RMSNorm (two roundings), rotate-half
    RoPE with dtype-cast coefficients and rounded products; V passes through."""
    dt = x.dtype
    M = x.size(0)
    heads = x.float().view(M, QH + 2 * KH, D)

    def one(h, w):
        n = _rt(h * torch.rsqrt((h * h).sum(-1, keepdim=True) / D + eps), dt)
        n = _rt(n * w.float(), dt)
        other = torch.roll(n, D // 2, -1)
        c = _rt(cos[positions.long()], dt).repeat(1, 2)[:, None, :]
        s = _rt(sin[positions.long()], dt).repeat(1, 2)[:, None, :]
        left, right = _rt(n * c, dt), _rt(other * s, dt)
        sign = torch.cat((-torch.ones(D // 2), torch.ones(D // 2)))
        return (left + sign * right).to(dt)

    q = one(heads[:, :QH], q_w)
    k = one(heads[:, QH:QH + KH], k_w)
    v = x.view(M, QH + 2 * KH, D)[:, QH + KH:].clone()
    return q.view(M, 1, QH, D), k.view(M, 1, KH, D), v.view(M, 1, KH, D)


def k_quantize_rows(x):
    """``lfm25_fp8.py:17-23``: ``scale=max(amax/448,1e-12)``; clamp; round to e4m3 (RNE)."""
    xf = x.float()
    scale = (xf.abs().amax(-1) / E4M3_MAX).clamp_min(1e-12)
    q = (xf / scale[:, None]).clamp(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)
    return q, scale


def k_rms_norm_fp8(x, weight, eps, residual=None):
    """``lfm25_fp8.py:27-41``: fused form equals norm followed by row quantisation."""
    out, summed = k_rms_norm(x, weight, eps, residual)
    q, s = k_quantize_rows(out)
    return q, s, summed


def k_swiglu_fp8(x):
    """``lfm25_fp8.py:45-54``."""
    return k_quantize_rows(k_swiglu(x))


def k_fp8_linear(xq, xs, wq, ws, dtype=torch.bfloat16):
    """Dequantised matmul that ``lfm25_fp8.py:77-105`` approximates; accumulated in float64 so the
    expectation itself carries no summation error."""
    return ((xq.double() @ wq.double().T) * xs.double()[:, None] * ws.double()[None, :]).to(dtype)


def k_store_kv(k, v):
    """Per (token, head) e4m3 rows and fp32 scales (``lfm25_fp8_kv.py:28-55``)."""
    def one(t):
        tf = t.float()
        s = (tf.abs().amax(-1) / E4M3_MAX).clamp_min(1e-12)
        return (tf / s[..., None]).clamp(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn), s
    (kq, ks), (vq, vs) = one(k), one(v)
    return kq, ks, vq, vs


def k_attend(q, k_hist, v_hist, length, scale, k_scales=None, v_scales=None):
    """One row of decode attention over ``[0, length)``: fp32 softmax over the
    (dequantised) history for every query head (``lfm25_fp8_kv.py:72-135`` /
    ``lfm25_engine.py:1562-1572``).  ``q [QH,D]``, history ``[T,KH,D]``."""
    QH, KH = q.size(0), k_hist.size(1)
    kf, vf = k_hist[:length].float(), v_hist[:length].float()
    if k_scales is not None:
        kf, vf = kf * k_scales[:length, :, None], vf * v_scales[:length, :, None]
    kf = kf.repeat_interleave(QH // KH, 1).permute(1, 0, 2)
    vf = vf.repeat_interleave(QH // KH, 1).permute(1, 0, 2)
    p = torch.softmax(torch.einsum("hd,htd->ht", q.float(), kf) * scale, -1)
    return torch.einsum("ht,htd->hd", p, vf)


def causal_attention(q, k, v, scale):
    """Causal GQA attention for one packed sequence ``[T,heads,D]`` in fp32 (library
    routine, ``lfm25_engine.py:1390-1394``)."""
    g = q.size(1) // k.size(1)
    o = F.scaled_dot_product_attention(q.float().permute(1, 0, 2)[None],
                                       k.float().repeat_interleave(g, 1).permute(1, 0, 2)[None],
                                       v.float().repeat_interleave(g, 1).permute(1, 0, 2)[None],
                                       is_causal=True, scale=scale)
    return o[0].permute(1, 0, 2)


# --------------------------------------------------------------------------- scheduler integer logic
def build_stop_table(pieces: Sequence[str], stops: Sequence[str]) -> torch.Tensor:
    """Prefix automaton of ``text_stops.py:17-39``; ``pieces[i]`` is the text of
    token ``i``.  Entry = next state + 65536 when a stop completed."""
    states = sorted({"", *(s[:i] for s in stops for i in range(1, len(s)))}, key=len)
    table = torch.zeros(len(states), len(pieces), dtype=torch.int32)
    for si, pre in enumerate(states):
        for ti, piece in enumerate(pieces):
            text = pre + piece
            hit = any(s in text for s in stops)
            nxt = max((j for j, p in enumerate(states) if text.endswith(p)), key=lambda j: len(states[j]))
            table[si, ti] = nxt + (65536 if hit else 0)
    return table


def record_sample_row(token, length, limit, state, table_row_value, eos, ignore_eos):
    """Finish code of ``lfm25_session.py:46-50``: 1 EOS, 2 stop, 3 length, 0 live."""
    if token == eos and not ignore_eos:
        return 1
    if table_row_value >= 65536:
        return 2
    return 3 if length + 1 >= limit else 0


def session_rng_key(seed: int, position: int) -> int:
    """Per-row key of ``lfm25_sampling.py:19-20``."""
    return ((seed & 0x7FFFFFFFFFFFFFFF) + position * 0x9E3779B97F4A7C15) & 0x7FFFFFFFFFFFFFFF
