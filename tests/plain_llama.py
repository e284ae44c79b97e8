"""A plain, slow implementation of the Llama dense decoder: whole sequences, no
cache, no batching, one function per part, written from the reference's formulas.
It shares no code with hfee_amd (it reads config.json and the safetensors file
through the `json` and `safetensors` libraries itself).

All arithmetic is float64 by default: the reference computes in float32 with
float64 in the spots named below, so float64 throughout differs from it by
float32 rounding only and serves both the 32-bit and the bfloat16 comparison.
"""
from __future__ import annotations

import json
import math
import os

import torch

F64 = torch.float64


def to_bfloat16(x: torch.Tensor) -> torch.Tensor:
    """x rounded to the nearest bfloat16 number (ties to even), as float64 again."""
    return x.to(torch.float32).to(torch.bfloat16).to(F64)


def same(x: torch.Tensor) -> torch.Tensor:
    return x


# ---------------------------------------------------------------- parts -----

def plain_rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """/root/reference/internal/ggml/ops.go:124-134: ss = sum x^2 (float64);
    scale = 1/sqrt(ss/len + eps); y = x * scale * weight.  eps is inside the
    square root, added to the mean."""
    x = x.to(F64)
    ss = (x * x).sum(dim=-1, keepdim=True)
    scale = 1.0 / torch.sqrt(ss / x.shape[-1] + float(eps))
    return x * scale * weight.to(F64)


def plain_matmul(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """/root/reference/internal/ggml/ops.go:54-71: out[t, r] = W[r, :] . x[t, :],
    W stored [out, in]."""
    return x.to(F64) @ w.to(F64).t()


def plain_rope_frequencies(head_dim: int, theta: float, scaling=None) -> torch.Tensor:
    """/root/reference/internal/llm/model.go:150-158: inv_freq[i] = 1/theta^(2i/dim),
    divided by a per-dimension factor when the file brings one.  The llama3 rule
    that makes those factors from config.json's rope_scaling: wavelengths shorter
    than N0/high keep their frequency, longer than N0/low are divided by `factor`,
    between the two the result slides linearly in N0/wavelength."""
    half = head_dim // 2
    inv = [1.0 / math.pow(theta, (2 * i) / head_dim) for i in range(half)]
    if scaling is not None:
        factor = float(scaling["factor"])
        lo = float(scaling["low_freq_factor"])
        hi = float(scaling["high_freq_factor"])
        n0 = float(scaling["original_max_position_embeddings"])
        out = []
        for f in inv:
            wavelen = 2 * math.pi / f
            if wavelen < n0 / hi:
                out.append(f)
            elif wavelen > n0 / lo:
                out.append(f / factor)
            else:
                s = (n0 / wavelen - lo) / (hi - lo)
                out.append((1 - s) * f / factor + s * f)
        inv = out
    return torch.tensor(inv, dtype=F64)


def plain_rope(x: torch.Tensor, positions, inv_freq: torch.Tensor, pairing: str = "half") -> torch.Tensor:
    """/root/reference/internal/llm/forward.go:180-196.  x: [T, heads, head_dim].
    For i < half: angle = pos * inv_freq[i]; pair (a, b) = (i, i+half) ("half") or
    (2i, 2i+1) ("interleaved"); x[a] <- x[a] cos - x[b] sin; x[b] <- x[a] sin + x[b] cos."""
    x = x.to(F64).clone()
    T, _, hd = x.shape
    half = inv_freq.numel()
    pos = torch.as_tensor(positions, dtype=F64, device=x.device).reshape(T, 1)
    ang = pos * inv_freq.to(x.device).reshape(1, half)          # [T, half]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    if pairing == "half":
        a = torch.arange(half, device=x.device)
        b = a + half
    elif pairing == "interleaved":
        a = 2 * torch.arange(half, device=x.device)
        b = a + 1
    else:
        raise ValueError(pairing)
    x0, x1 = x[:, :, a].clone(), x[:, :, b].clone()
    x[:, :, a] = x0 * cos - x1 * sin
    x[:, :, b] = x0 * sin + x1 * cos
    return x


def plain_softmax(s: torch.Tensor) -> torch.Tensor:
    """/root/reference/internal/ggml/ops.go:136-150: subtract the maximum,
    exponentiate, divide by the sum (along the last dimension)."""
    s = s.to(F64)
    e = torch.exp(s - s.max(dim=-1, keepdim=True).values)
    return e / e.sum(dim=-1, keepdim=True)


def plain_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float | None = None,
                    window: int = 0, positions=None, round_terms=None) -> torch.Tensor:
    """/root/reference/internal/llm/forward.go:144-178.  q: [T, H, hd], k, v:
    [T, K, hd] (k already rotated).  Head h reads KV head h // (H/K); token i
    scores keys 0..i (no mask values: the range is the mask), score = dot * scale,
    softmax, weighted sum of v.  `window` > 0 narrows the range to the last
    `window` keys (the reference has no window; 0 is its behaviour).  round_terms
    (not in the reference): a function that the terms exp(score - max) go through
    on their way into the weighted sum, while their sum is taken unrounded, as an
    engine does that multiplies in a narrow format and divides by a float32 sum."""
    T, H, hd = q.shape
    K = k.shape[1]
    group = H // K
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    q, k, v = q.to(F64), k.to(F64), v.to(F64)
    out = torch.zeros(T, H, hd, dtype=F64, device=q.device)
    for i in range(T):
        lo = 0 if window <= 0 else max(0, i - window + 1)
        # the heads of a group side by side: qi[kvh, g] is head kvh * group + g, which reads KV head kvh
        qi = q[i].reshape(K, group, hd)
        scores = torch.einsum("nkd,kgd->kgn", k[lo:i + 1], qi) * scale
        if round_terms is None:
            p = plain_softmax(scores)
            out[i] = torch.einsum("kgn,nkd->kgd", p, v[lo:i + 1]).reshape(H, hd)
        else:
            e = torch.exp(scores - scores.max(dim=-1, keepdim=True).values)
            out[i] = (torch.einsum("kgn,nkd->kgd", round_terms(e), v[lo:i + 1]) / e.sum(dim=-1, keepdim=True)).reshape(H, hd)
    return out


def plain_swiglu(gate: torch.Tensor, up: torch.Tensor, activation: str = "silu") -> torch.Tensor:
    """/root/reference/internal/ggml/ops.go:159-165: g / (1 + exp(-g)) * up.  The other
    activations (config.json's `hidden_act`; the reference has the SiLU alone, so they are pinned
    by the library's own functions in test_plain.py): gelu = g/2 (1 + erf(g / sqrt 2)),
    gelu_pytorch_tanh = g/2 (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))), relu = max(g, 0)."""
    g = gate.to(F64)
    if activation == "silu":
        a = g / (1 + torch.exp(-g))
    elif activation == "gelu":
        a = 0.5 * g * (1 + torch.erf(g / math.sqrt(2.0)))
    elif activation == "gelu_pytorch_tanh":
        a = 0.5 * g * (1 + torch.tanh(math.sqrt(2.0 / math.pi) * (g + 0.044715 * g ** 3)))
    elif activation == "relu":
        a = torch.clamp(g, min=0)
    else:
        raise ValueError(f"hidden_act {activation!r}")
    return a * up.to(F64)


# ---------------------------------------------------------------- model -----

class PlainLlama:
    """Reads a model folder; forward(tokens) -> logits [T, vocab] (float64)."""

    def __init__(self, model_dir: str, round_like_engine: bool = False, device: str = "cpu", weights=None):
        """weights: the tensors of another PlainLlama of the same folder, to share (read only).  device: where torch keeps the tensors and does the arithmetic (the same
        float64 library routines either way).  round_like_engine (not in the reference): what a bfloat16 engine keeps in
        bfloat16 between its kernels is rounded to bfloat16 here too (the normed
        stream, q and k after the rotation, v, the terms of the softmax on their way
        into the weighted sum, the attention's output, the gated product); sums
        stay float64 and the stream itself is not rounded.  The distance of an
        engine to this twin is what its kernels add beyond the format."""
        from safetensors import safe_open
        self.r = to_bfloat16 if round_like_engine else same
        with open(os.path.join(model_dir, "config.json"), "r", encoding="utf-8") as f:
            c = json.load(f)
        self.c = c
        self.d = c["hidden_size"]
        self.L = c["num_hidden_layers"]
        self.H = c["num_attention_heads"]
        self.K = c.get("num_key_value_heads") or self.H
        self.hd = c.get("head_dim") or self.d // self.H
        self.eps = c.get("rms_norm_eps", 1e-5)
        self.tied = bool(c.get("tie_word_embeddings", False))
        self.act = c.get("hidden_act", "silu")
        scaling = c.get("rope_scaling")
        if scaling is not None and scaling.get("rope_type", scaling.get("type")) != "llama3":
            scaling = None
        self.inv_freq = plain_rope_frequencies(self.hd, c.get("rope_theta", 10000.0), scaling)
        self.device = device
        if weights is not None:
            self.w = weights
            return
        self.w = {}
        with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt") as f:
            for name in f.keys():
                self.w[name] = f.get_tensor(name).to(device=device).to(F64)

    def embed(self, tokens) -> torch.Tensor:
        """/root/reference/internal/llm/forward.go:75-77: the token's row of the table,
        as it is stored (no scaling by sqrt(width) or anything else)."""
        return self.w["model.embed_tokens.weight"][torch.as_tensor(tokens, dtype=torch.long, device=self.device)]

    def attention_sublayer(self, x, l, pos, kv=None, window=0):
        """/root/reference/internal/llm/forward.go:82-107: what the attention half of
        layer l adds to the stream x [T, d] at positions pos: norm first, then q/k/v,
        rotation of q and k, attention, output projection.  Returns (delta, (k, v));
        with kv given, those keys and values are read instead of made."""
        w, T = self.w, x.shape[0]
        p = f"model.layers.{l}."
        r = self.r
        xb = r(plain_rmsnorm(x, w[p + "input_layernorm.weight"], self.eps))            # forward.go:82
        q = plain_matmul(xb, w[p + "self_attn.q_proj.weight"]).reshape(T, self.H, self.hd)
        q = r(plain_rope(q, pos, self.inv_freq))                                       # forward.go:96-97
        if kv is None:
            k = plain_matmul(xb, w[p + "self_attn.k_proj.weight"]).reshape(T, self.K, self.hd)
            v = plain_matmul(xb, w[p + "self_attn.v_proj.weight"]).reshape(T, self.K, self.hd)
            kv = (r(plain_rope(k, pos, self.inv_freq)), r(v))                          # forward.go:99-101
        att = plain_attention(q, kv[0], kv[1], window=window,
                              round_terms=None if r is same else r).reshape(T, self.H * self.hd)    # forward.go:104
        return plain_matmul(r(att), w[p + "self_attn.o_proj.weight"]), kv              # forward.go:106

    def feed_forward_sublayer(self, x, l):
        """/root/reference/internal/llm/forward.go:109-113: what the feed-forward half
        of layer l adds to the stream: norm first, then down(silu(gate) * up) (or the
        activation that config.json names instead of the SiLU)."""
        w = self.w
        p = f"model.layers.{l}."
        xb = self.r(plain_rmsnorm(x, w[p + "post_attention_layernorm.weight"], self.eps))    # forward.go:109
        h = plain_swiglu(plain_matmul(xb, w[p + "mlp.gate_proj.weight"]),
                         plain_matmul(xb, w[p + "mlp.up_proj.weight"]), self.act)      # forward.go:110-112
        return plain_matmul(self.r(h), w[p + "mlp.down_proj.weight"])                  # forward.go:113

    def block(self, x, l, pos, kv=None, window=0):
        """/root/reference/internal/llm/forward.go:80-115: x <- x + attention(norm(x));
        x <- x + feed_forward(norm(x)): each half reads the normed stream and adds to
        the stream itself.  Returns (x, (k, v))."""
        delta, kv = self.attention_sublayer(x, l, pos, kv, window)
        x = x + delta                                                                  # forward.go:107
        x = x + self.feed_forward_sublayer(x, l)                                       # forward.go:114
        return x, kv

    def head(self, x) -> torch.Tensor:
        """/root/reference/internal/llm/forward.go:124-141: the final norm, then the
        product with the output matrix (the embedding table itself when tied,
        model.go:118-121); nothing scales the logits."""
        w = self.w
        x = self.r(plain_rmsnorm(x, w["model.norm.weight"], self.eps))                 # forward.go:124-128
        head = w["model.embed_tokens.weight"] if self.tied else w["lm_head.weight"]    # model.go:118-121
        return plain_matmul(x, head)                                                   # forward.go:132-141

    def forward(self, tokens, schedule=None, windows=None, rows=None) -> torch.Tensor:
        """/root/reference/internal/llm/forward.go:51-142 for one sequence from
        position 0, logits at every position (or at the positions `rows` only: the
        reference runs its final norm and head for the wanted rows, forward.go:117-130).  schedule: [(layer, cache, writes)] in
        running order (default: every layer once, its own cache); an entry that does
        not write reads the keys and values that the entry which wrote `cache` made.
        windows: {layer: keys kept} for layers with a window."""
        T = len(tokens)
        pos = list(range(T))
        x = self.embed(tokens)
        if schedule is None:
            schedule = [(l, l, True) for l in range(self.L)]
        windows = windows or {}
        caches = {}
        for l, cache, writes in schedule:
            x, kv = self.block(x, l, pos, None if writes else caches[cache], windows.get(l, 0))
            if writes:
                caches[cache] = kv
        if rows is not None:
            x = x[torch.as_tensor(list(rows), dtype=torch.long, device=self.device)]
        return self.head(x).cpu()

    def greedy(self, prompt, n_new: int) -> list:
        """Greedy continuation: first maximum wins (/root/reference/internal/llm/sampler.go:76-84)."""
        toks = list(prompt)
        out = []
        for _ in range(n_new):
            logits = self.forward(toks)[-1]
            nxt = plain_argmax(logits)
            out.append(nxt)
            toks.append(nxt)
        return out


# -------------------------------------------------------------- sampler -----

def plain_argmax(logits) -> int:
    """/root/reference/internal/llm/sampler.go:76-84: strict '>' keeps the first maximum."""
    best = 0
    vals = logits.tolist()
    for i, v in enumerate(vals):
        if v > vals[best]:
            best = i
    return best


def plain_repeat_penalty(logits: torch.Tensor, history, penalty: float, last_n: int) -> torch.Tensor:
    """/root/reference/internal/llm/sampler.go:57-74: each distinct id in the last
    `last_n` ids (all if last_n < 0): logit > 0 -> / penalty, else * penalty."""
    logits = logits.clone()
    if penalty == 1 or last_n == 0:
        return logits
    recent = list(history)
    if last_n > 0 and len(recent) > last_n:
        recent = recent[-last_n:]
    for i in set(recent):
        if i >= logits.numel():
            continue
        logits[i] = logits[i] / penalty if logits[i] > 0 else logits[i] * penalty
    return logits


def plain_sampling_distribution(logits: torch.Tensor, temperature: float, top_k: int = 0,
                                top_p: float = 1.0, min_p: float = 0.0) -> torch.Tensor:
    """/root/reference/internal/llm/sampler.go:86-129 up to the draw: the
    probability of every id (zeros outside the kept set).  Candidates are the
    top_k largest in descending order; prob = exp((logit - max)/T) normalised;
    top_p keeps the shortest prefix whose cumulative probability reaches it;
    min_p cuts at the first candidate below min_p * prob[0]; the draw is
    proportional to the kept probabilities."""
    V = logits.numel()
    k = V if top_k <= 0 or top_k > V else top_k
    l32 = logits.to(torch.float32)
    order = torch.argsort(l32, descending=True, stable=True)[:k]
    cl = l32[order]
    probs = torch.exp(((cl - cl[0]) / torch.tensor(temperature, dtype=torch.float32)).to(F64))
    probs = probs / probs.sum()
    keep = k
    if 0 < top_p < 1:
        cum = torch.cumsum(probs, 0)
        # compare against the float32 value of top_p widened, as the reference does
        hit = (cum >= float(torch.tensor(top_p, dtype=torch.float32))).nonzero()
        if hit.numel():
            keep = int(hit[0]) + 1
    if min_p > 0:
        thr = float(torch.tensor(min_p, dtype=torch.float32)) * probs[0]
        for i in range(1, keep):
            if probs[i] < thr:
                keep = i
                break
    dist = torch.zeros(V, dtype=F64)
    dist[order[:keep]] = probs[:keep] / probs[:keep].sum()
    return dist
