"""A plain, slow implementation of the Llama / Qwen2 / Qwen3 dense decoder.

Whole sequences, no cache, NumPy float64, one function for each part.  It shares
no code with the package under test: it reads config.json with ``json`` and the
weights with the ``safetensors`` library, and every formula is written out from
the reference's text (paths relative to the reference's ``src/dotnet``).

The reference stores Q/K rows permuted for interleaved rotary pairs (GGUF
convention); checkpoints in the config.json + safetensors convention are not
permuted and need the split-half pairing, which the reference describes in
Daisi.Llogos.Cpu/Rope.cs:65-76.  Both pairings are here; a test shows they are
the same function up to that row permutation.
"""
from __future__ import annotations

import json
import math
import os

import numpy as np


# --------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------

def embedding(table: np.ndarray, tokens) -> np.ndarray:
    """x = E[token]: a row copy without scaling.
    Daisi.Llogos/Inference/ForwardPass.cs:205; Daisi.Llogos.Cpu/CpuBackend.cs:327-339."""
    return np.asarray(table, dtype=np.float64)[np.asarray(tokens, dtype=np.int64)]


def linear(x: np.ndarray, w: np.ndarray, b: np.ndarray | None = None) -> np.ndarray:
    """y = x . W^T with W stored [out_features, in_features].
    Daisi.Llogos/Inference/ForwardPass.cs:890-895 (K = dim0, N = dim1);
    vectors in tests/Daisi.Llogos.Tests/Cpu/MathOpsTests.cs:10-28."""
    y = np.asarray(x, dtype=np.float64) @ np.asarray(w, dtype=np.float64).T
    if b is not None:
        y = y + np.asarray(b, dtype=np.float64)
    return y


def rms_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """out_i = x_i * (1 / sqrt(mean(x^2) + eps)) * w_i; eps inside the root, the
    weight multiplies as it is.  Daisi.Llogos.Cpu/RmsNorm.cs:14-65."""
    x = np.asarray(x, dtype=np.float64)
    inv = 1.0 / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)
    return x * inv * np.asarray(w, dtype=np.float64)


def per_head_rms_norm(x: np.ndarray, w: np.ndarray, n_heads: int, head_dim: int, eps: float) -> np.ndarray:
    """RMSNorm over each head's head_dim values, one weight vector [head_dim]
    shared by all heads.  Daisi.Llogos.Cpu/CpuBackend.cs:406-421."""
    t = x.shape[0]
    xh = np.asarray(x, dtype=np.float64).reshape(t, n_heads, head_dim)
    inv = 1.0 / np.sqrt((xh * xh).mean(axis=-1, keepdims=True) + eps)
    return (xh * inv * np.asarray(w, dtype=np.float64)).reshape(t, n_heads * head_dim)


def rope_frequencies(rot_dim: int, theta: float) -> np.ndarray:
    """f_i = 1 / theta^(2i / rot_dim), in double.  Daisi.Llogos.Cpu/Rope.cs:145-162."""
    i = np.arange(rot_dim // 2, dtype=np.float64)
    return 1.0 / np.power(float(theta), 2.0 * i / rot_dim)


def llama3_frequency_factors(freqs: np.ndarray, factor: float, low_freq_factor: float,
                             high_freq_factor: float, original_max_position: int) -> np.ndarray:
    """Per-pair divisors for the reference's frequency-factor table (the effective frequency is
    f_i / factor_i, Daisi.Llogos.Cpu/Rope.cs:42-63; the reference takes the table from the
    checkpoint, here the Llama-3 rule fills it from the configuration).

    The rule, stated by how often a pair turns within the original context, r_i =
    original * f_i / (2 pi): pairs that turn more than `high` times keep their frequency;
    pairs that turn less than `low` times run `factor` times slower; between the two the new
    frequency is a mix of the slowed and the kept one, f_i * ((1 - s) / factor + s), with
    s = (r_i - low) / (high - low) going from 0 to 1 across the band.  The mix is linear in the
    *frequency* (that is in 1 / factor), not in the divisor."""
    f = np.asarray(freqs, dtype=np.float64)
    turns = float(original_max_position) * f / (2.0 * math.pi)
    s = np.clip((turns - low_freq_factor) / (high_freq_factor - low_freq_factor), 0.0, 1.0)
    kept_share = np.where(turns > high_freq_factor, 1.0, np.where(turns < low_freq_factor, 0.0, s))
    new_f = f * ((1.0 - kept_share) / float(factor) + kept_share)
    return f / new_f


def rope_split_half(x: np.ndarray, positions, n_heads: int, head_dim: int, freqs: np.ndarray) -> np.ndarray:
    """Rotate the pair (x[i], x[i + rot/2]) of every head by angle pos * f_i;
    dimensions at and beyond rot = 2 * len(freqs) pass through.
    Daisi.Llogos.Cpu/Rope.cs:115-129 (pairing), :147-152 (angle in double)."""
    t = x.shape[0]
    half = len(freqs)
    xh = np.array(x, dtype=np.float64).reshape(t, n_heads, head_dim)
    ang = np.asarray(positions, dtype=np.float64)[:, None] * freqs[None, :]
    cos, sin = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    x0 = xh[:, :, :half].copy()
    x1 = xh[:, :, half:2 * half].copy()
    xh[:, :, :half] = x0 * cos - x1 * sin
    xh[:, :, half:2 * half] = x0 * sin + x1 * cos
    return xh.reshape(t, n_heads * head_dim)


def rope_interleaved(x: np.ndarray, positions, n_heads: int, head_dim: int, freqs: np.ndarray) -> np.ndarray:
    """The reference's default pairing (x[2i], x[2i+1]).  Daisi.Llogos.Cpu/Rope.cs:147-162."""
    t = x.shape[0]
    half = len(freqs)
    xh = np.array(x, dtype=np.float64).reshape(t, n_heads, head_dim)
    ang = np.asarray(positions, dtype=np.float64)[:, None] * freqs[None, :]
    cos, sin = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    x0 = xh[:, :, 0:2 * half:2].copy()
    x1 = xh[:, :, 1:2 * half:2].copy()
    xh[:, :, 0:2 * half:2] = x0 * cos - x1 * sin
    xh[:, :, 1:2 * half:2] = x0 * sin + x1 * cos
    return xh.reshape(t, n_heads * head_dim)


def softmax(s: np.ndarray) -> np.ndarray:
    """Stable softmax over the last axis.  Daisi.Llogos.Cpu/Softmax.cs:8-30."""
    s = np.asarray(s, dtype=np.float64)
    m = s.max(axis=-1, keepdims=True)
    e = np.exp(s - m)
    return e / e.sum(axis=-1, keepdims=True)


def visible(q_pos: int, k_pos: int, window: int = 0, sinks: int = 0) -> bool:
    """Which keys a query sees.  Causal: key position <= query position
    (Daisi.Llogos.Cuda/kernels/composite_ops.cu:412-413).  With a window the cache keeps
    the first `sinks` positions and the last `window` ones
    (Daisi.Llogos/Inference/AttentionStrategy.cs:46-71)."""
    if k_pos > q_pos:
        return False
    if window <= 0:
        return True
    return k_pos < sinks or k_pos > q_pos - window


def attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, n_heads: int, n_kv_heads: int,
              head_dim: int, scale: float | None = None, window: int = 0, sinks: int = 0,
              positions=None, rows=None) -> np.ndarray:
    """Causal grouped-query attention over one whole sequence.  Query head h reads
    KV head h // (n_heads / n_kv_heads); score = (q . k) * scale with scale =
    1/sqrt(head_dim) applied after the dot; softmax over the visible keys; o = sum p v.
    Daisi.Llogos.Cpu/CpuBackend.cs:476-590 (group :510, scale :541, sum guard :581).
    rows: the queries to work out (all by default; the other rows of the result stay zero)."""
    t = q.shape[0]
    if scale is None:
        scale = 1.0 / math.sqrt(head_dim)
    if positions is None:
        positions = list(range(t))
    qh = np.asarray(q, dtype=np.float64).reshape(t, n_heads, head_dim)
    kh = np.asarray(k, dtype=np.float64).reshape(t, n_kv_heads, head_dim)
    vh = np.asarray(v, dtype=np.float64).reshape(t, n_kv_heads, head_dim)
    group = n_heads // n_kv_heads
    out = np.zeros((t, n_heads, head_dim), dtype=np.float64)
    for h in range(n_heads):
        g = h // group
        for i in (range(t) if rows is None else rows):
            keys = [j for j in range(t) if visible(positions[i], positions[j], window, sinks)]
            s = (kh[keys, g, :] @ qh[i, h, :]) * scale
            p = softmax(s)
            out[i, h, :] = p @ vh[keys, g, :]
    return out.reshape(t, n_heads * head_dim)


def silu(z: np.ndarray) -> np.ndarray:
    """silu(z) = z / (1 + exp(-z)).  Daisi.Llogos.Cpu/Silu.cs:9-16."""
    z = np.asarray(z, dtype=np.float64)
    return z / (1.0 + np.exp(-z))


def swiglu_mlp(x: np.ndarray, w_gate: np.ndarray, w_up: np.ndarray, w_down: np.ndarray) -> np.ndarray:
    """d = (silu(x Wg^T) * (x Wu^T)) Wd^T, no biases.
    Daisi.Llogos/Inference/ForwardPass.cs:240-246."""
    return linear(silu(linear(x, w_gate)) * linear(x, w_up), w_down)


# --------------------------------------------------------------------------
# configuration and weights, read independently of the package
# --------------------------------------------------------------------------

ARCH_DEFAULTS = {
    # architecture name -> (qkv bias, per-head qk norm); the reference finds both by tensor
    # presence (Daisi.Llogos/Model/ModelLoader.cs:106-110).
    "LlamaForCausalLM": (False, False),
    "Qwen2ForCausalLM": (True, False),
    "Qwen3ForCausalLM": (False, True),
}


class PlainConfig:
    def __init__(self, d: dict):
        arch = d["architectures"][0]
        bias_default, qk_norm = ARCH_DEFAULTS[arch]
        self.arch = arch
        self.n_layers = int(d["num_hidden_layers"])
        self.hidden = int(d["hidden_size"])
        self.intermediate = int(d["intermediate_size"])
        self.vocab = int(d["vocab_size"])
        self.n_heads = int(d["num_attention_heads"])
        self.n_kv_heads = int(d.get("num_key_value_heads", self.n_heads))
        self.head_dim = int(d.get("head_dim") or self.hidden // self.n_heads)
        self.eps = float(d.get("rms_norm_eps", 1e-6))
        self.theta = float(d.get("rope_theta", 10000.0))
        self.rot_dim = int(self.head_dim * float(d.get("partial_rotary_factor", 1.0)))
        self.rope_scaling = d.get("rope_scaling")
        self.bias = bool(d.get("attention_bias", bias_default))
        self.qk_norm = qk_norm
        self.tied = bool(d.get("tie_word_embeddings", False))
        self.windows = [0] * self.n_layers
        if d.get("use_sliding_window") and d.get("sliding_window"):
            first = int(d.get("max_window_layers", 0))
            for i in range(first, self.n_layers):
                self.windows[i] = int(d["sliding_window"])

    def frequencies(self) -> np.ndarray:
        f = rope_frequencies(self.rot_dim, self.theta)
        rs = self.rope_scaling
        kind = rs.get("rope_type", rs.get("type")) if rs else None
        if kind == "llama3":
            f = f / llama3_frequency_factors(f, float(rs["factor"]), float(rs["low_freq_factor"]),
                                             float(rs["high_freq_factor"]),
                                             int(rs["original_max_position_embeddings"]))
        elif kind == "linear":
            # one factor for every pair in the reference's per-pair table, f_i / factor_i (Cpu/Rope.cs:42-63):
            # positions are stretched by `factor`
            f = f / float(rs["factor"])
        elif kind not in (None, "default"):
            raise ValueError(f"unknown rotary scaling '{kind}'")
        return f


def load_folder(folder: str):
    """config.json -> PlainConfig, model.safetensors -> {name: float64 array}."""
    import torch
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as fh:
        cfg = PlainConfig(json.load(fh))
    raw = load_file(os.path.join(folder, "model.safetensors"))
    weights = {k: v.to(torch.float64).numpy() for k, v in raw.items()}
    return cfg, weights


# --------------------------------------------------------------------------
# the whole model
# --------------------------------------------------------------------------

def decoder_layer(cfg: PlainConfig, w: dict, i: int, x: np.ndarray, positions, freqs: np.ndarray,
                  window: int | None = None, sinks: int = 0) -> np.ndarray:
    """One block: x += attn(norm1(x)); x += mlp(norm2(x)).  The reference defers the second
    add into the next layer's fused norm (Daisi.Llogos/Inference/ForwardPass.cs:214-252);
    written out here.  Order inside attention: projections (:368-370), per-head norm
    (:372-376), bias (:379-382; a bias belongs to its projection, no checkpoint has both),
    rotation (:385), attention (:391-401), output projection (:404)."""
    p = f"model.layers.{i}."
    n = rms_norm(x, w[p + "input_layernorm.weight"], cfg.eps)
    q = linear(n, w[p + "self_attn.q_proj.weight"], w.get(p + "self_attn.q_proj.bias"))
    k = linear(n, w[p + "self_attn.k_proj.weight"], w.get(p + "self_attn.k_proj.bias"))
    v = linear(n, w[p + "self_attn.v_proj.weight"], w.get(p + "self_attn.v_proj.bias"))
    if cfg.qk_norm:
        q = per_head_rms_norm(q, w[p + "self_attn.q_norm.weight"], cfg.n_heads, cfg.head_dim, cfg.eps)
        k = per_head_rms_norm(k, w[p + "self_attn.k_norm.weight"], cfg.n_kv_heads, cfg.head_dim, cfg.eps)
    q = rope_split_half(q, positions, cfg.n_heads, cfg.head_dim, freqs)
    k = rope_split_half(k, positions, cfg.n_kv_heads, cfg.head_dim, freqs)
    win = cfg.windows[i] if window is None else window
    a = attention(q, k, v, cfg.n_heads, cfg.n_kv_heads, cfg.head_dim, window=win, sinks=sinks,
                  positions=positions)
    x = x + linear(a, w[p + "self_attn.o_proj.weight"])
    n = rms_norm(x, w[p + "post_attention_layernorm.weight"], cfg.eps)
    x = x + swiglu_mlp(n, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                       w[p + "mlp.down_proj.weight"])
    return x


def forward(cfg: PlainConfig, w: dict, tokens, window: int | None = None, sinks: int = 0) -> np.ndarray:
    """Logits [len(tokens), vocab] of one whole sequence that starts at position 0.
    Final norm and head: Daisi.Llogos/Inference/ForwardPass.cs:179-180; the head is the
    embedding when there is no output tensor (Daisi.Llogos/Model/ModelWeights.cs:29)."""
    positions = list(range(len(tokens)))
    freqs = cfg.frequencies()
    x = embedding(w["model.embed_tokens.weight"], tokens)
    for i in range(cfg.n_layers):
        x = decoder_layer(cfg, w, i, x, positions, freqs, window, sinks)
    n = rms_norm(x, w["model.norm.weight"], cfg.eps)
    head = w["model.embed_tokens.weight"] if (cfg.tied or "lm_head.weight" not in w) else w["lm_head.weight"]
    return linear(n, head)


def forward_many(cfg: PlainConfig, get, sequences) -> list:
    """forward() for several sequences of a model too large to hold in float64: `get(name)`
    reads one tensor (float64) when it is needed, and a layer's tensors are read once for all
    sequences.  The same functions in the same order as forward()."""
    freqs = cfg.frequencies()
    table = get("model.embed_tokens.weight")
    xs = [embedding(table, t) for t in sequences]
    names = ["input_layernorm.weight", "post_attention_layernorm.weight", "self_attn.q_proj.weight",
             "self_attn.k_proj.weight", "self_attn.v_proj.weight", "self_attn.o_proj.weight", "mlp.gate_proj.weight",
             "mlp.up_proj.weight", "mlp.down_proj.weight"]
    if cfg.bias:
        names += ["self_attn.q_proj.bias", "self_attn.k_proj.bias", "self_attn.v_proj.bias"]
    if cfg.qk_norm:
        names += ["self_attn.q_norm.weight", "self_attn.k_norm.weight"]
    for i in range(cfg.n_layers):
        p = f"model.layers.{i}."
        w = {p + n: get(p + n) for n in names}
        xs = [decoder_layer(cfg, w, i, x, list(range(len(t))), freqs) for x, t in zip(xs, sequences)]
        del w
    head = table if cfg.tied else get("lm_head.weight")
    norm_w = get("model.norm.weight")
    return [linear(rms_norm(x, norm_w, cfg.eps), head) for x in xs]


# --------------------------------------------------------------------------
# sampling
# --------------------------------------------------------------------------

def argmax_first(values) -> int:
    """First maximum wins (strict >).  Daisi.Llogos/Inference/Sampler.cs:234-247."""
    best, best_val = 0, values[0]
    for i in range(1, len(values)):
        if values[i] > best_val:
            best, best_val = i, values[i]
    return best


def sample(logits, u: float, temperature: float = 0.8, top_k: int = 40, top_p: float = 0.95,
           repetition_penalty: float = 1.1, frequency_penalty: float = 0.0, presence_penalty: float = 0.0,
           min_p: float = 0.0, typical_p: float = 1.0, penalty_count: int = 64, min_keep: int = 1,
           penalize_newline: bool = False, history=(), candidates_out=None,
           intervals_out=None) -> int:
    """The reference's pipeline, Daisi.Llogos/Inference/Sampler.cs:26-85, with the uniform
    draw `u` given by the caller: penalties (:89-143), greedy short cut (:56-57), temperature
    (:60-62), top-k (:249-276), min-p (:157-174), softmax over candidates (:278-295),
    typical-p (:182-230), top-p (:297-332), draw (:334-345).  float32 as in the reference.
    candidates_out: a list that receives the ids the draw chooses among (every id some `u` gives);
    intervals_out: a dict that receives id -> (lo, hi), the part of [0, 1) whose `u` draw that id."""
    work = np.array(logits, dtype=np.float32)
    n = len(work)
    f32 = np.float32
    if not (repetition_penalty == 1.0 and frequency_penalty == 0 and presence_penalty == 0):
        hist = list(history)
        if 0 < penalty_count < len(hist):
            hist = hist[len(hist) - penalty_count:]
        newline = (10, 13)
        if repetition_penalty != 1.0:
            for t in hist:
                if not 0 <= t < n or (not penalize_newline and t in newline):
                    continue
                work[t] = work[t] / f32(repetition_penalty) if work[t] > 0 else work[t] * f32(repetition_penalty)
        if frequency_penalty != 0 or presence_penalty != 0:
            counts = {}
            for t in hist:
                counts[t] = counts.get(t, 0) + 1
            for t, c in counts.items():
                if not 0 <= t < n or (not penalize_newline and t in newline):
                    continue
                work[t] -= f32(frequency_penalty) * f32(c)
                work[t] -= f32(presence_penalty)
    if temperature == 0:
        if candidates_out is not None:
            candidates_out.append(argmax_first(work))
        if intervals_out is not None:
            intervals_out[argmax_first(work)] = (0.0, 1.0)
        return argmax_first(work)
    work = work * (f32(1.0) / f32(temperature))
    k = top_k if 0 < top_k < n else n
    order = sorted(range(n), key=lambda i: (-work[i], i))   # insertion with strict > keeps index order on ties
    cand = order[:k]
    keep = max(min_keep, 1)
    if 0 < min_p < 1.0 and len(cand) > keep:
        thr = max(work[c] for c in cand) + f32(math.log(min_p))
        kept = []
        for c in cand:
            if work[c] >= thr or len(kept) < keep:
                kept.append(c)
        cand = kept
    m = max(work[c] for c in cand)
    probs = np.zeros(n, dtype=np.float32)
    for c in cand:
        probs[c] = np.exp(work[c] - m, dtype=np.float32)
    probs /= probs[cand].sum(dtype=np.float32)
    if 0 < typical_p < 1.0 and len(cand) > keep:
        ent = -sum(float(probs[c]) * math.log(float(probs[c])) for c in cand if probs[c] > 0)
        scored = sorted(cand, key=lambda c: abs((-math.log(float(probs[c])) if probs[c] > 0 else 3.4e38) - ent))
        kept, cum = [], 0.0
        for c in scored:
            kept.append(c)
            cum += float(probs[c])
            if cum >= typical_p and len(kept) >= keep:
                break
        s = sum(float(probs[c]) for c in kept)
        if s > 0:
            for c in cand:
                if c not in kept:
                    probs[c] = 0
            for c in kept:
                probs[c] = f32(probs[c] / s)
        cand = kept
    if 0 < top_p < 1.0:
        cand = sorted(cand, key=lambda c: -probs[c])
        cum, cutoff = 0.0, len(cand)
        for i, c in enumerate(cand):
            cum += float(probs[c])
            if cum > top_p and i + 1 >= keep:
                cutoff = i + 1
                break
        cand = cand[:cutoff]
        s = sum(float(probs[c]) for c in cand)
        if s > 0:
            for c in cand:
                probs[c] = f32(probs[c] / s)
    if candidates_out is not None:
        candidates_out.extend(cand)
    if intervals_out is not None:
        lo = 0.0
        for c in cand:
            intervals_out[c] = (lo, lo + float(probs[c]))
            lo += float(probs[c])
    cum = 0.0
    for c in cand:
        cum += float(probs[c])
        if u < cum:
            return c
    return cand[0]


def generate_greedy(cfg: PlainConfig, w: dict, prompt, max_new_tokens: int, stop=()) -> list:
    """Prefill, then sample / stop check / append / forward; a sampled stop token ends the
    sequence and is not emitted.  Daisi.Llogos/Inference/TextGenerator.cs:46-115."""
    seq = list(prompt)
    out = []
    for _ in range(max_new_tokens):
        tok = argmax_first(forward(cfg, w, seq)[-1])
        if tok in stop:
            break
        out.append(tok)
        seq.append(tok)
    return out
