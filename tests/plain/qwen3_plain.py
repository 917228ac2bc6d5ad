"""Plain, slow, whole-sequence Qwen3 in torch: the oracle of the test-suite.

No cache, no batching, no kernels, one function per part, nothing imported from
the product package.  Every function follows the reference's formula and cites
it (paths relative to the reference checkout).  Runs in float32 (or float64 for a
tighter oracle) on the device the weights live on: the CPU, or, for the sizes of real
models, the GPU with torch's plain float32 products (``use_exact_float32_products``).
"""
from __future__ import annotations

import json
import math
from pathlib import Path

import torch


# --------------------------------------------------------------------------- config
def read_config(folder) -> dict:
    """Config numbers exactly as the reference reads them: jllm/model/qwen3.py:37-56."""
    c = json.loads((Path(folder) / "config.json").read_text())
    nq = c["num_attention_heads"]
    return dict(
        vocab_size=c["vocab_size"],
        hidden_size=c["hidden_size"],
        intermediate_size=c["intermediate_size"],
        num_hidden_layers=c["num_hidden_layers"],
        num_heads=nq,
        num_kv_heads=c.get("num_key_value_heads", nq),
        head_dim=c.get("head_dim", c["hidden_size"] // nq),
        rms_norm_eps=c["rms_norm_eps"],
        rope_theta=c.get("rope_theta", 1_000_000.0),
        tie_word_embeddings=c.get("tie_word_embeddings", False),
    )


def read_weights(folder, dtype=torch.float32) -> dict:
    """All tensors of all shards, by name, cast to one dtype: jllm/model/weights.py:21-37."""
    from safetensors.torch import load_file

    out = {}
    for shard in sorted(Path(folder).glob("*.safetensors")):
        for k, v in load_file(str(shard)).items():
            out[k] = v.to(dtype)
    return out


def use_exact_float32_products() -> None:
    """Forbid torch's reduced-precision modes for float32 matrix products on the GPU, so that
    the oracle there is the same arithmetic as on the CPU (up to summation order)."""
    torch.backends.cuda.matmul.allow_tf32 = False
    torch.backends.cudnn.allow_tf32 = False
    torch.set_float32_matmul_precision("highest")


# --------------------------------------------------------------------------- parts
def embed(table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """Row gather, no scaling: jllm/model/common.py:35-36."""
    return table[ids]


def linear(weight: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """x @ W.T with W stored [out, in], no bias for Qwen3: jllm/model/common.py:39-41."""
    return x @ weight.T


def rms_norm(weight: torch.Tensor, eps: float, x: torch.Tensor) -> torch.Tensor:
    """x * rsqrt(mean(x^2, last axis) + eps) * w: jllm/model/common.py:44-48."""
    inv_rms = torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return (x * inv_rms) * weight


def rope_cos_sin(dim: int, theta: float, positions: torch.Tensor, dtype):
    """inv_freq[i] = theta^(-2i/dim); angles = pos * inv_freq; the half-table is
    repeated twice along the last axis: jllm/model/common.py:51-55."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.float32) / dim))
    freqs = positions.to(torch.float32)[..., None] * inv_freq.to(positions.device)
    emb = torch.cat([freqs, freqs], dim=-1)
    return torch.cos(emb).to(dtype), torch.sin(emb).to(dtype)


def rotate_half(u: torch.Tensor) -> torch.Tensor:
    """(u1, u2) -> (-u2, u1) on the two halves of the last axis: jllm/model/common.py:58-60."""
    u1, u2 = torch.chunk(u, 2, dim=-1)
    return torch.cat([-u2, u1], dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x*cos + rotate_half(x)*sin, cos/sin broadcast over heads: jllm/model/common.py:63-66.
    x is [heads, T, D]; cos, sin are [T, D]."""
    return x * cos[None] + rotate_half(x) * sin[None]


def swiglu(w_gate, w_up, w_down, x):
    """down(silu(gate(x)) * up(x)): jllm/model/common.py:75-76."""
    return linear(w_down, torch.nn.functional.silu(linear(w_gate, x)) * linear(w_up, x))


def causal_mask(t_q: int, t_k: int, device=None) -> torch.Tensor:
    """Key j is visible to query i iff j <= (t_k - t_q) + i: jllm/model/common.py:203-214
    (with every row valid); for t_q == t_k this is the tril of common.py:163."""
    q_idx = torch.arange(t_q, device=device)[:, None]
    k_idx = torch.arange(t_k, device=device)[None, :]
    return k_idx <= (t_k - t_q) + q_idx


def attention_core(q, k, v, mask):
    """Scores (q.k) / sqrt(D), masked with -inf, softmax over keys, times v; kv heads
    are repeated so that q head h reads kv head h // (nq/nkv):
    jllm/model/common.py:173-178 and :191-200.  q [nq,Tq,D], k,v [nkv,Tk,D]."""
    nq, nkv, d = q.shape[0], k.shape[0], q.shape[-1]
    rep = nq // nkv
    out = []
    for h in range(nq):      # head by head: the scores of a long sequence are [T, T] floats per head
        scores = (q[h] @ k[h // rep].T) * (1.0 / math.sqrt(d))
        scores = torch.where(mask, scores, torch.full_like(scores, float("-inf")))
        out.append(torch.softmax(scores, dim=-1) @ v[h // rep])
    return torch.stack(out)


def attention_block(w: dict, p: str, cfg: dict, x: torch.Tensor, positions: torch.Tensor, window=None,
                    shared_kv=None, return_kv=False):
    """Projections, per-head q/k RMSNorm over D before RoPE, RoPE, causal attention,
    head-major concat, output projection: jllm/model/common.py:114-137; q/k norm
    :107-111 with the model's rms_norm_eps (jllm/model/weights.py:128-129).
    Beyond the reference, for tests of the engine's generality: ``window`` keeps only the last
    ``window`` keys visible, ``shared_kv`` makes the block read another block's (k, v)."""
    t = x.shape[0]
    nq, nkv, d = cfg["num_heads"], cfg["num_kv_heads"], cfg["head_dim"]
    q = linear(w[f"{p}.q_proj.weight"], x).reshape(t, nq, d).transpose(0, 1)
    q = rms_norm(w[f"{p}.q_norm.weight"], cfg["rms_norm_eps"], q)
    cos, sin = rope_cos_sin(d, cfg["rope_theta"], positions, x.dtype)
    q = apply_rope(q, cos, sin)
    if shared_kv is None:
        k = linear(w[f"{p}.k_proj.weight"], x).reshape(t, nkv, d).transpose(0, 1)
        v = linear(w[f"{p}.v_proj.weight"], x).reshape(t, nkv, d).transpose(0, 1)
        k = rms_norm(w[f"{p}.k_norm.weight"], cfg["rms_norm_eps"], k)
        k = apply_rope(k, cos, sin)
    else:
        k, v = shared_kv
    mask = causal_mask(t, t, x.device)
    if window:
        idx = torch.arange(t, device=x.device)
        mask = mask & (idx[None, :] > idx[:, None] - window)
    out = attention_core(q, k, v, mask)
    out = out.transpose(0, 1).reshape(t, nq * d)
    out = linear(w[f"{p}.o_proj.weight"], out)
    return (out, (k, v)) if return_kv else out


def decoder_layer(w: dict, i: int, cfg: dict, h: torch.Tensor, positions: torch.Tensor):
    """Pre-norm residual block: h += attn(norm(h)); h += mlp(norm(h)):
    jllm/model/common.py:140-147."""
    p = f"model.layers.{i}"
    eps = cfg["rms_norm_eps"]
    h = h + attention_block(
        w, f"{p}.self_attn", cfg, rms_norm(w[f"{p}.input_layernorm.weight"], eps, h), positions
    )
    m = rms_norm(w[f"{p}.post_attention_layernorm.weight"], eps, h)
    h = h + swiglu(
        w[f"{p}.mlp.gate_proj.weight"], w[f"{p}.mlp.up_proj.weight"], w[f"{p}.mlp.down_proj.weight"], m
    )
    return h


def forward(w: dict, cfg: dict, token_ids, first_position: int = 0, rows=None) -> torch.Tensor:
    """Whole-sequence forward of one request, logits at every position [T, V] (or only at the
    positions ``rows``, as the reference's engine applies the head to the wanted rows only,
    jllm/engine/generate.py:140-142): jllm/model/common.py:150-170.  lm_head is the embedding
    table when tied (jllm/model/weights.py:143-146).  Runs where the weights are."""
    device = w["model.embed_tokens.weight"].device
    ids = torch.as_tensor(token_ids, dtype=torch.long, device=device)
    positions = torch.arange(ids.shape[0], device=device) + first_position
    h = embed(w["model.embed_tokens.weight"], ids)
    for i in range(cfg["num_hidden_layers"]):
        h = decoder_layer(w, i, cfg, h, positions)
    if rows is not None:
        h = h[torch.as_tensor(rows, dtype=torch.long, device=device)]
    h = rms_norm(w["model.norm.weight"], cfg["rms_norm_eps"], h)
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    return linear(head, h)


def greedy_generate(w: dict, cfg: dict, prompt, max_new_tokens: int, eos_id=None):
    """argmax of the last position's logits, re-running the whole sequence each time;
    stops after max_new_tokens or once eos is emitted (it is emitted and counted):
    jllm/engine/generate.py:142 and jllm/engine/engine.py:507-512."""
    seq = list(prompt)
    out = []
    for _ in range(max_new_tokens):
        tok = int(torch.argmax(forward(w, cfg, seq)[-1]))
        out.append(tok)
        seq.append(tok)
        if eos_id is not None and tok == eos_id:
            break
    return out


def softmax_temperature(logits: torch.Tensor, temperature: float) -> torch.Tensor:
    """Distribution that temperature sampling draws from: softmax(logits / T) in float32."""
    return torch.softmax(logits.to(torch.float32) / temperature, dim=-1)


def forward_scheduled(w: dict, cfg: dict, token_ids, schedule, windows=None) -> torch.Tensor:
    """Whole-sequence forward with the layers run in a given order: ``schedule`` is a list of
    (layer index, index of the earlier entry whose keys/values it reads, or None); ``windows``
    maps a layer index to its attention window.  With schedule [(0, None), (1, None), ...] and
    no windows this is ``forward``."""
    ids = torch.as_tensor(token_ids, dtype=torch.long)
    positions = torch.arange(ids.shape[0])
    eps = cfg["rms_norm_eps"]
    h = embed(w["model.embed_tokens.weight"], ids)
    kvs = []
    for layer, cache_of in schedule:
        p = f"model.layers.{layer}"
        a, kv = attention_block(
            w, f"{p}.self_attn", cfg, rms_norm(w[f"{p}.input_layernorm.weight"], eps, h), positions,
            window=(windows or {}).get(layer), shared_kv=None if cache_of is None else kvs[cache_of], return_kv=True)
        kvs.append(kv)
        h = h + a
        m = rms_norm(w[f"{p}.post_attention_layernorm.weight"], eps, h)
        h = h + swiglu(w[f"{p}.mlp.gate_proj.weight"], w[f"{p}.mlp.up_proj.weight"], w[f"{p}.mlp.down_proj.weight"], m)
    h = rms_norm(w["model.norm.weight"], eps, h)
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    return linear(head, h)
