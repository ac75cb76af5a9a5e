"""Each part alone against its plain counterpart, the order of layers as data (a layer run
twice, a layer reading another's cache), and toy parts defined here that are registered, built
and stepped without a change to the library's files: a mixer with state of its own, a
feed-forward with a router and experts, and another position encoding."""
import dataclasses
import importlib
import math
import os

import numpy as np
import pytest
import torch

import gpu_helpers as H
import plain_model as pm
import tiny_configs as tc

pytestmark = pytest.mark.gpu
L = H.llogos
P = importlib.import_module("daisi-llogos_amd.parts")
K = importlib.import_module("daisi-llogos_amd.ops.kernels")
DEV = torch.device("cuda:0")
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 2e-5, "bfloat16": 1e-2}


def _np(t):
    return t.detach().cpu().double().numpy()


def _rand(rng, shape, dtype, scale=1.0):
    t = torch.tensor(rng.standard_normal(shape) * scale, dtype=DT[dtype])
    return t, t.double().numpy()


def _ctx(rt, lens, new, slots=None):
    B, T = len(lens), sum(new)
    tok_seq = np.repeat(np.arange(B), new).astype(np.int32)
    tok_pos = np.concatenate([np.arange(l - n, l) for l, n in zip(lens, new)]).astype(np.int32)
    i32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=DEV)
    return P.StepContext(runtime=rt, n_tokens=T, batch=B, ids=i32(np.zeros(T)), tok_seq=i32(tok_seq),
                         tok_pos=i32(tok_pos), slots=i32(slots or list(range(B))),
                         cu_seqlens=np.concatenate([[0], np.cumsum(new)]).tolist(),
                         starts=[l - n for l, n in zip(lens, new)], slot_ids=slots or list(range(B)),
                         is_decode=max(new) == 1, max_context=max(lens),
                         cu_dev=i32(np.concatenate([[0], np.cumsum(new)])))


@pytest.mark.parametrize("dtype", H.DTYPES)
def test_linear_stacks_matrices_by_rows(dtype):
    rng = np.random.default_rng(0)
    rt = P.Runtime(DEV, DT[dtype])
    wa, wa_ = _rand(rng, (24, 40), dtype, 0.1)
    wb, wb_ = _rand(rng, (8, 40), dtype, 0.1)
    ba, ba_ = _rand(rng, (24,), dtype)
    bb, bb_ = _rand(rng, (8,), dtype)
    lin = P.Linear(["a", "b"], 40, [24, 8], bias=True)
    assert [(s.name, s.shape, s.kind) for s in lin.tensor_specs()] == [
        ("a.weight", (24, 40), "matrix"), ("a.bias", (24,), "bias"), ("b.weight", (8, 40), "matrix"),
        ("b.bias", (8,), "bias")]
    lin.bind({"a.weight": wa, "b.weight": wb, "a.bias": ba, "b.bias": bb}.get, rt)
    x, x_ = _rand(rng, (5, 40), dtype)
    want = np.concatenate([pm.linear(x_, wa_, ba_), pm.linear(x_, wb_, bb_)], axis=1)
    assert np.abs(_np(lin.forward(x.to(DEV))) - want).max() <= TOL[dtype] * 3
    assert np.abs(_np(lin.forward(x.to(DEV), rows_out=24)) - want[:, :24]).max() <= TOL[dtype] * 3
    assert lin.bias.dtype == torch.float32 and lin.weight.dtype == DT[dtype]


@pytest.mark.parametrize("dtype", H.DTYPES)
def test_rmsnorm_part(dtype):
    rng = np.random.default_rng(1)
    rt = P.Runtime(DEV, DT[dtype])
    w, w_ = _rand(rng, (72,), dtype)
    norm = P.RMSNorm("n", 72, 3e-4)
    norm.bind({"n.weight": w}.get, rt)
    x = torch.tensor(rng.standard_normal((6, 72)), dtype=torch.float32, device=DEV)
    x_ = _np(x)
    d, d_ = _rand(rng, (6, 72), dtype)
    out = norm.forward(x, d.to(DEV))
    assert np.abs(_np(out) - pm.rms_norm(x_ + d_, w_, 3e-4)).max() <= TOL[dtype] * 3
    assert np.abs(_np(x) - (x_ + d_)).max() < 1e-6                      # the residual stream took the sum


def test_rotary_part_tables():
    rt = P.Runtime(DEV, torch.float32)
    plain_f = pm.rope_frequencies(24, 5e5)
    rot = P.Rotary(48, 24, 5e5)
    assert np.allclose(rot.freqs, plain_f, rtol=1e-15)
    sc = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
              original_max_position_embeddings=64)
    rot3 = P.Rotary(48, 24, 5e5, scaling=sc)
    want = plain_f / pm.llama3_frequency_factors(plain_f, 8.0, 1.0, 4.0, 64)
    assert np.allclose(rot3.freqs, want, rtol=1e-15) and not np.allclose(want, plain_f)
    assert np.allclose(P.Rotary(48, 24, 5e5, scaling=dict(rope_type="linear", factor=4.0)).freqs, plain_f / 4)
    rot3.bind(lambda n: None, rt)
    ctx = _ctx(rt, [70, 3], [5, 3])
    cs = _np(rot3.prepare(ctx))
    ang = _np(ctx.tok_pos)[:, None] * want[None, :]
    assert np.abs(cs[..., 0] - np.cos(ang)).max() < 1e-7 and np.abs(cs[..., 1] - np.sin(ang)).max() < 1e-7
    assert rot3.prepare(ctx) is rot3.prepare(ctx)                       # made once per step
    with pytest.raises(ValueError):
        P.Rotary(48, 50, 1e4)
    with pytest.raises(ValueError):
        P.Rotary(48, 24, 1e4, scaling=dict(rope_type="yarn", factor=2.0))


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("nh,nkv,hd,bias,qk_norm,window", [(4, 2, 16, True, False, 0), (6, 1, 32, False, True, 0),
                                                           (5, 5, 48, True, True, 20)])
def test_attention_part_alone(dtype, nh, nkv, hd, bias, qk_norm, window):
    """The mixer alone: a prompt in one step, then two single tokens, against plain parts."""
    rng = np.random.default_rng(2)
    rt = P.Runtime(DEV, DT[dtype])
    hidden, T = 40, 70
    rot = P.Rotary(hd, hd, 1e4)
    att = P.Attention("a.", hidden, nh, nkv, hd, rot, bias=bias, qk_norm=qk_norm, eps=1e-5, window=window)
    tensors, plain = {}, {}
    for spec in att.tensor_specs():
        scale = 0.2 if spec.kind == "matrix" else 1.0
        t, a = _rand(rng, spec.shape, dtype, scale)
        if spec.kind == "norm":
            t = (1 + 0.1 * t.float()).to(DT[dtype]); a = t.double().numpy()
        tensors[spec.name], plain[spec.name] = t, a
    att.bind(tensors.get, rt)
    assert att.kv_spec() == P.KVSpec(nkv, hd, window, 0) and att.state_spec() is None
    x, x_ = _rand(rng, (T, hidden), dtype)
    # plain: projections, norm, rotation, attention, output projection
    q = pm.linear(x_, plain["a.q_proj.weight"], plain.get("a.q_proj.bias"))
    k = pm.linear(x_, plain["a.k_proj.weight"], plain.get("a.k_proj.bias"))
    v = pm.linear(x_, plain["a.v_proj.weight"], plain.get("a.v_proj.bias"))
    if qk_norm:
        q = pm.per_head_rms_norm(q, plain["a.q_norm.weight"], nh, hd, 1e-5)
        k = pm.per_head_rms_norm(k, plain["a.k_norm.weight"], nkv, hd, 1e-5)
    f = pm.rope_frequencies(hd, 1e4)
    q, k = pm.rope_split_half(q, range(T), nh, hd, f), pm.rope_split_half(k, range(T), nkv, hd, f)
    want = pm.linear(pm.attention(q, k, v, nh, nkv, hd, window=window), plain["a.o_proj.weight"])
    # engine part, with a cache of its own
    pool = lambda: torch.zeros((3, nkv, 64 * hd), dtype=DT[dtype], device=DEV)
    cache = P.LayerCache(k_pool=pool(), v_pool=pool(), table=torch.tensor([[2, 0]], dtype=torch.int32, device=DEV))
    plain_out = lambda o: K.sum_parts(o, None, DT[dtype])            # a mixer may hand on partial sums
    outs = [plain_out(att.forward(_ctx(rt, [68], [68]), x[:68].to(DEV), cache))]
    for t in (68, 69):
        outs.append(plain_out(att.forward(_ctx(rt, [t + 1], [1]), x[t:t + 1].to(DEV), cache)))
    got = _np(torch.cat(outs))
    assert np.abs(got - want).max() <= TOL[dtype] * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("hd", [128, 64])
@pytest.mark.parametrize("nh,nkv,bias,qk_norm,window", [(8, 2, True, True, 0), (16, 1, False, False, 0),
                                                        (5, 5, False, True, 70), (12, 4, True, False, 0)])
@pytest.mark.parametrize("lens", [[62, 130, 5], [700, 380, 5]])
def test_single_token_steps_from_the_projection_in_one_kernel(nh, nkv, bias, qk_norm, window, hd, lens, monkeypatch):
    """Head sizes 128 and 64 in bfloat16: the attention kernel that makes its queries and the
    step's key and value from the projection itself gives, bit for bit, the outputs and the cache
    pages of the rotation kernel followed by the attention kernel, across a page's end, and both
    agree with the plain parts.  With the longer sequences the attention takes several blocks along
    the context, whose results a second kernel merges."""
    dtype, hidden = "bfloat16", 72
    rng = np.random.default_rng(nh)
    rt = P.Runtime(DEV, DT[dtype])
    att = P.Attention("a.", hidden, nh, nkv, hd, P.Rotary(hd, hd, 1e4), bias=bias, qk_norm=qk_norm, eps=1e-5,
                      window=window)
    tensors, plain = {}, {}
    for spec in att.tensor_specs():
        t, a = _rand(rng, spec.shape, dtype, 0.2 if spec.kind == "matrix" else 1.0)
        if spec.kind == "norm":
            t = (1 + 0.1 * t.float()).to(DT[dtype]); a = t.double().numpy()
        tensors[spec.name], plain[spec.name] = t, a
    att.bind(tensors.get, rt)
    taken = []
    fused_kernel = K.attention_decode_fused
    monkeypatch.setattr(K, "attention_decode_fused", lambda *a, **k: (taken.append(fused_kernel(*a, **k)), taken[-1])[1])
    steps = 4
    xs = [_rand(rng, (l + steps, hidden), dtype) for l in lens]
    width = (max(lens) + steps + 63) // 64 + 1
    table = torch.tensor(rng.permutation(3 * width).reshape(3, width), dtype=torch.int32, device=DEV)
    results = []
    for fused in (False, True):
        att.fuse_decode = fused
        pool = lambda: torch.full((3 * width, nkv, 64 * hd), float("nan"), dtype=DT[dtype], device=DEV)
        cache = P.LayerCache(k_pool=pool(), v_pool=pool(), table=table)
        x0 = torch.cat([x[:l] for (x, _), l in zip(xs, lens)]).to(DEV)
        outs = [K.sum_parts(att.forward(_ctx(rt, lens, lens), x0, cache), None, DT[dtype])]
        for t in range(steps):
            xt = torch.stack([x[l + t] for (x, _), l in zip(xs, lens)]).to(DEV)
            outs.append(K.sum_parts(att.forward(_ctx(rt, [l + t + 1 for l in lens], [1] * 3), xt, cache), None, DT[dtype]))
        results.append((torch.cat(outs), cache.k_pool.clone(), cache.v_pool.clone()))
    assert len(taken) == steps and all(t is not None for t in taken)       # the fused kernel took every single-token step
    for a, b in zip(*results):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))       # bit for bit, NaN of unwritten pages included
    # against the plain parts, sequence by sequence
    got = _np(results[1][0])
    o = sum(lens)
    for i, ((_, x_), l) in enumerate(zip(xs, lens)):
        q = pm.linear(x_, plain["a.q_proj.weight"], plain.get("a.q_proj.bias"))
        k = pm.linear(x_, plain["a.k_proj.weight"], plain.get("a.k_proj.bias"))
        v = pm.linear(x_, plain["a.v_proj.weight"], plain.get("a.v_proj.bias"))
        if qk_norm:
            q = pm.per_head_rms_norm(q, plain["a.q_norm.weight"], nh, hd, 1e-5)
            k = pm.per_head_rms_norm(k, plain["a.k_norm.weight"], nkv, hd, 1e-5)
        f = pm.rope_frequencies(hd, 1e4)
        n = l + steps
        q, k = pm.rope_split_half(q, range(n), nh, hd, f), pm.rope_split_half(k, range(n), nkv, hd, f)
        want = pm.linear(pm.attention(q, k, v, nh, nkv, hd, window=window), plain["a.o_proj.weight"])
        for t in range(steps):
            row = got[o + 3 * t + i]
            assert np.abs(row - want[l + t]).max() <= TOL[dtype] * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("dtype", H.DTYPES)
def test_swiglu_part_alone(dtype):
    rng = np.random.default_rng(3)
    rt = P.Runtime(DEV, DT[dtype])
    ffn = P.SwiGLU("m.", 40, 72)
    tensors, plain = {}, {}
    for spec in ffn.tensor_specs():
        tensors[spec.name], plain[spec.name] = _rand(rng, spec.shape, dtype, 0.2)
    ffn.bind(tensors.get, rt)
    x, x_ = _rand(rng, (9, 40), dtype)
    want = pm.swiglu_mlp(x_, plain["m.gate_proj.weight"], plain["m.up_proj.weight"], plain["m.down_proj.weight"])
    got = K.sum_parts(ffn.forward(None, x.to(DEV)), None, DT[dtype])
    assert np.abs(_np(got) - want).max() <= TOL[dtype] * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("T", [37, 200])
@pytest.mark.parametrize("dtype", H.DTYPES)
def test_block_arrangement_alone(dtype, T):
    """The pre-norm block built from its parts: the pending sum handed in is added by the first
    norm, the mixer's output by the second, and the feed-forward's output is handed on (or, in bfloat16,
    added by the product that made it: the one-pass product for a single token, the library's epilogue for
    a prompt of more than 128 rows); against the plain layer of the first tiny configuration, a prompt and
    then a single token."""
    name = "tiny_a"
    cfg, w = H.plain(name)
    rt = P.Runtime(DEV, DT[dtype])
    models = importlib.import_module("daisi-llogos_amd.models")
    arch = L.architecture_of(tc.ALL[name])
    spec = arch.model_spec(arch.read_config(tc.ALL[name]))
    block = models.model.build_layer(spec.layers[1])
    from safetensors.torch import load_file
    tensors = load_file(os.path.join(H.folder(name), "model.safetensors"))
    block.bind(tensors.get, rt)
    rng = np.random.default_rng(12)
    x0, pend = rng.standard_normal((T + 1, cfg.hidden)), rng.standard_normal((T + 1, cfg.hidden)) * 0.3
    f = cfg.frequencies()
    want = pm.decoder_layer(cfg, w, 1, x0 + pend, list(range(T + 1)), f)
    kv = block.mixer.kv_spec()
    pool = lambda: torch.zeros((6, kv.n_kv_heads, 64 * kv.head_dim), dtype=DT[dtype], device=DEV)
    cache = P.LayerCache(k_pool=pool(), v_pool=pool(),
                         table=torch.tensor([[1, 4, 2, 5]], dtype=torch.int32, device=DEV))
    got = []
    for lo, hi in ((0, T), (T, T + 1)):
        x = torch.tensor(x0[lo:hi], dtype=torch.float32, device=DEV)
        p = torch.tensor(pend[lo:hi], dtype=torch.float32, device=DEV)
        x_out, pending = block.forward(_ctx(rt, [hi], [hi - lo]), x, p, cache)
        assert x_out is x                                                # the stream is updated in place
        if isinstance(pending, K.RowSquares):                            # the last product has added itself
            assert dtype == "bfloat16"
            if pending.sums is not None:                                 # few rows: with the rows' sums of squares
                assert hi - lo <= K.RESIDUAL_MAX_ROWS
                squares = _np(pending.sums).sum(0)[: hi - lo]
                assert np.allclose(squares, (_np(x_out) ** 2).sum(1), rtol=1e-5)
            else:
                assert hi - lo > 128
            got.append(_np(x_out))
        else:
            got.append(_np(x_out) + _np(K.sum_parts(pending, None, torch.float32)))
    got = np.concatenate(got)
    tol = 1e-4 if dtype == "float32" else TOL[dtype] * max(1.0, np.abs(want).max())
    assert np.abs(got - want).max() <= tol


# ---------------------------------------------------------------------------
# the order of layers is data
# ---------------------------------------------------------------------------
def _scheduled_arch(name, schedule):
    models = importlib.import_module("daisi-llogos_amd.models")

    def spec(cfg, **kw):
        s = L.dense_decoder_spec(cfg, **kw)
        s.schedule = [models.ScheduleEntry(l, c) for l, c in schedule]
        return s
    L.register_architecture(name, L.ARCHITECTURES["Qwen2ForCausalLM"].read_config, spec)


def _plain_scheduled(cfg, w, tokens, schedule):
    """Plain forward in which the order of layers is a list; an entry may read the keys and
    values another entry made."""
    T = len(tokens)
    f = cfg.frequencies()
    x = pm.embedding(w["model.embed_tokens.weight"], tokens)
    kv = {}
    for e, (i, src) in enumerate(schedule):
        p = f"model.layers.{i}."
        n = pm.rms_norm(x, w[p + "input_layernorm.weight"], cfg.eps)
        q = pm.rope_split_half(pm.linear(n, w[p + "self_attn.q_proj.weight"], w.get(p + "self_attn.q_proj.bias")),
                               range(T), cfg.n_heads, cfg.head_dim, f)
        if src is None:
            k = pm.rope_split_half(pm.linear(n, w[p + "self_attn.k_proj.weight"], w.get(p + "self_attn.k_proj.bias")),
                                   range(T), cfg.n_kv_heads, cfg.head_dim, f)
            v = pm.linear(n, w[p + "self_attn.v_proj.weight"], w.get(p + "self_attn.v_proj.bias"))
            kv[e] = (k, v)
        else:
            k, v = kv[src]
        a = pm.attention(q, k, v, cfg.n_heads, cfg.n_kv_heads, cfg.head_dim)
        x = x + pm.linear(a, w[p + "self_attn.o_proj.weight"])
        n = pm.rms_norm(x, w[p + "post_attention_layernorm.weight"], cfg.eps)
        x = x + pm.swiglu_mlp(n, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return pm.linear(pm.rms_norm(x, w["model.norm.weight"], cfg.eps), w["lm_head.weight"])


@pytest.mark.parametrize("dtype", H.DTYPES)
def test_a_layer_twice_and_a_layer_reading_anothers_cache(tmp_path, dtype):
    schedule = [(0, None), (1, None), (1, None), (0, 0)]        # layer 1 twice; layer 0 again on entry 0's cache
    _scheduled_arch("ScheduledToyForCausalLM", schedule)
    cfg_json = dict(tc.TINY_A, architectures=["ScheduledToyForCausalLM"])
    folder = L.write_random_model(str(tmp_path / "m"), cfg_json, seed=4)
    import json
    from safetensors.torch import load_file
    pcfg = pm.PlainConfig(dict(tc.TINY_A))
    w = {k: v.double().numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    toks = list(H.tokens("tiny_a", 80, 5))
    want = _plain_scheduled(pcfg, w, toks, schedule)
    eng = L.Engine.from_folder(folder, dtype=dtype, max_tokens=256)
    assert len(eng.cache.groups) == 1 and eng.cache.groups[0].k.shape[0] == 3      # three caches for four runs
    s = eng.alloc_slot()
    rows = [_np(eng.step([(s, toks[:66])], want="all"))] + [_np(eng.step([(s, [t])])) for t in toks[66:]]
    H.close(np.concatenate(rows), want, dtype, "scheduled layers", config="tiny_a")
    models = importlib.import_module("daisi-llogos_amd.models")
    spec = L.dense_decoder_spec(L.ARCHITECTURES["Qwen2ForCausalLM"].read_config(tc.TINY_A))
    spec.schedule = [models.ScheduleEntry(0), models.ScheduleEntry(1, cache_of=1)]
    with pytest.raises(ValueError, match="before"):
        L.Model(spec)


# ---------------------------------------------------------------------------
# a toy mixer with state of its own, defined here
# ---------------------------------------------------------------------------
@P.register_mixer("toy_running_mean")
class RunningMean(P.Mixer):
    """out_t = W . mean(h_0 .. h_t): the running sum is the sequence's fixed-size state."""

    def __init__(self, prefix, hidden):
        self.prefix, self.hidden = prefix, hidden

    def tensor_specs(self):
        return [P.TensorSpec(self.prefix + "mix.weight", (self.hidden, self.hidden), "matrix")]

    def state_spec(self):
        return P.StateSpec((self.hidden,), torch.float32)

    def bind(self, get, rt):
        self.rt = rt
        self.w = get(self.prefix + "mix.weight").to(device=rt.device, dtype=torch.float32)

    def forward(self, ctx, h, cache):
        out = torch.empty_like(h)
        for b in range(ctx.batch):
            lo, hi = ctx.cu_seqlens[b], ctx.cu_seqlens[b + 1]
            slot = ctx.slot_ids[b]
            run = torch.cumsum(h[lo:hi].float(), 0) + cache.state[slot]
            cache.state[slot] = run[-1]
            count = torch.arange(ctx.starts[b] + 1, ctx.starts[b] + hi - lo + 1, device=h.device)[:, None]
            out[lo:hi] = ((run / count) @ self.w.T).to(h.dtype)
        return out


@dataclasses.dataclass(frozen=True)
class ToyConfig:
    vocab_size: int
    hidden_size: int
    n_layers: int
    architecture: str = "ToyStateForCausalLM"


def _toy_spec(cfg, **kw):
    models = importlib.import_module("daisi-llogos_amd.models")
    rot = P.Rotary(16, 16, 1e4)
    layers = []
    for i in range(cfg.n_layers):
        p = f"layers.{i}."
        mixer = ("toy_running_mean", dict(prefix=p, hidden=cfg.hidden_size)) if i % 2 == 0 else \
            ("attention", dict(prefix=p + "attn.", hidden=cfg.hidden_size, n_heads=2, n_kv_heads=1, head_dim=16,
                               position=rot))
        layers.append(models.LayerSpec(
            mixer=mixer, ffn=("swiglu", dict(prefix=p + "ffn.", hidden=cfg.hidden_size, intermediate=56)),
            mixer_norm=("rmsnorm", dict(name=p + "n1", width=cfg.hidden_size, eps=1e-6)),
            ffn_norm=("rmsnorm", dict(name=p + "n2", width=cfg.hidden_size, eps=1e-6))))
    return models.ModelSpec(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, embed_name="embed.weight",
                            layers=layers, final_norm=("rmsnorm", dict(name="norm", width=cfg.hidden_size, eps=1e-6)),
                            head_name="head", tie_head=False)


L.register_architecture("ToyStateForCausalLM",
                        lambda d: ToyConfig(d["vocab_size"], d["hidden_size"], d["n_layers"]), _toy_spec)


def _plain_toy(w, tokens, n_layers):
    T = len(tokens)
    x = pm.embedding(w["embed.weight"], tokens)
    f = pm.rope_frequencies(16, 1e4)
    for i in range(n_layers):
        p = f"layers.{i}."
        n = pm.rms_norm(x, w[p + "n1.weight"], 1e-6)
        if i % 2 == 0:
            a = pm.linear(np.cumsum(n, axis=0) / np.arange(1, T + 1)[:, None], w[p + "mix.weight"])
        else:
            q = pm.rope_split_half(pm.linear(n, w[p + "attn.q_proj.weight"]), range(T), 2, 16, f)
            k = pm.rope_split_half(pm.linear(n, w[p + "attn.k_proj.weight"]), range(T), 1, 16, f)
            a = pm.linear(pm.attention(q, k, pm.linear(n, w[p + "attn.v_proj.weight"]), 2, 1, 16), w[p + "attn.o_proj.weight"])
        x = x + a
        n = pm.rms_norm(x, w[p + "n2.weight"], 1e-6)
        x = x + pm.swiglu_mlp(n, w[p + "ffn.gate_proj.weight"], w[p + "ffn.up_proj.weight"], w[p + "ffn.down_proj.weight"])
    return pm.linear(pm.rms_norm(x, w["norm.weight"], 1e-6), w["head.weight"])


def test_a_toy_mixer_with_state_is_registered_built_and_stepped(tmp_path):
    from safetensors.torch import load_file
    cfg = {"architectures": ["ToyStateForCausalLM"], "vocab_size": 90, "hidden_size": 40, "n_layers": 3,
           "torch_dtype": "float32"}
    folder = L.write_random_model(str(tmp_path / "toy"), cfg, seed=2)
    w = {k: v.double().numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    eng = L.Engine.from_folder(folder, dtype="float32", max_tokens=512, n_slots=2)
    needs = eng.model.cache_needs()
    assert [st is not None for _, st in needs] == [True, False, True]
    assert [kv is not None for kv, _ in needs] == [False, True, False]
    rng = np.random.default_rng(0)
    seqs = [rng.integers(0, 90, size=n).tolist() for n in (30, 7, 75)]
    want = [_plain_toy(w, s, 3) for s in seqs]
    # whole and alone
    for s, wnt in zip(seqs, want):
        slot = eng.alloc_slot()
        H.close(_np(eng.step([(slot, s)], want="all")), wnt, "float32", "toy whole")
        eng.free_slot(slot)
    # a batch of unequal lengths, prompts then one token each; shorter ones end earlier; slots were used before,
    # so a state that is not zeroed when its slot is handed out again would show
    slots = [eng.alloc_slot() for _ in seqs]
    cut = [20, 3, 70]
    out = eng.step([(sl, s[:c]) for sl, s, c in zip(slots, seqs, cut)], want="all")
    rows = [[] for _ in seqs]
    o = 0
    for i, c in enumerate(cut):
        rows[i].append(_np(out[o:o + c])); o += c
    fed = list(cut)
    live = [0, 1, 2]
    while live:
        for i in [i for i in live if fed[i] == len(seqs[i])]:
            eng.free_slot(slots[i]); live.remove(i)
        if not live:
            break
        out = eng.step([(slots[i], [seqs[i][fed[i]]]) for i in live], want="last")
        for j, i in enumerate(live):
            rows[i].append(_np(out[j:j + 1])); fed[i] += 1
    for i in range(3):
        H.close(np.concatenate(rows[i]), want[i], "float32", f"toy batch seq {i}")
    with pytest.raises(L.CacheError, match="state"):
        s = eng.alloc_slot(); eng.step([(s, [1, 2, 3])]); eng.cache.truncate(s, 1)


def test_the_command_line_runs_a_toy_architecture(tmp_path, capsys):
    """The command line describes and runs a model from what the built model says of itself: the toy
    configuration has none of the dense decoder's fields."""
    cli = importlib.import_module("daisi-llogos_amd.__main__")
    from safetensors.torch import load_file
    cfg = {"architectures": ["ToyStateForCausalLM"], "vocab_size": 90, "hidden_size": 40, "n_layers": 3,
           "torch_dtype": "float32"}
    folder = L.write_random_model(str(tmp_path / "toy"), cfg, seed=2)
    w = {k: v.double().numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    prompt = [5, 17, 3, 80, 41]
    assert cli.main(["--model", folder, "--prompt", " ".join(map(str, prompt)), "-n", "6", "-t", "0",
                     "--repeat-penalty", "1.0", "--dtype", "float32", "--max-context", "64"]) == 0
    io = capsys.readouterr()
    assert "Loaded ToyStateForCausalLM: 3 layers, hidden 40, 2/1 heads, vocab 90" in io.err
    got = [int(t) for t in io.out.split()]
    seq = list(prompt)
    for _ in range(6):
        seq.append(int(np.argmax(_plain_toy(w, seq, 3)[-1])))
    assert got == seq[len(prompt):]


# ---------------------------------------------------------------------------
# a toy feed-forward with routing and a toy position encoding, defined here
# ---------------------------------------------------------------------------
@P.register_norm("toy_layernorm")
class ToyLayerNorm(P.Norm):
    """(v - mean(v)) / sqrt(var(v) + eps) * w + b with v = x + delta: a norm that is no scale of the whole row,
    written against the plain interface (a tensor or nothing as delta)."""

    def __init__(self, name, width, eps):
        self.name, self.width, self.eps = name, width, eps

    def tensor_specs(self):
        return [P.TensorSpec(self.name + ".weight", (self.width,), "norm"), P.TensorSpec(self.name + ".bias", (self.width,), "bias")]

    def bind(self, get, rt):
        self.rt = rt
        self.w = get(self.name + ".weight").to(device=rt.device, dtype=torch.float32)
        self.b = get(self.name + ".bias").to(device=rt.device, dtype=torch.float32)

    def forward(self, x, delta=None, rows=None, write_back=True):
        assert delta is None or isinstance(delta, torch.Tensor)
        v = x
        if delta is not None:
            v = x + (delta.float().sum(0) if delta.dim() == 3 else delta.float())
            if write_back:
                x.copy_(v)
        if rows is not None:
            v = v[rows.long()]
        out = torch.nn.functional.layer_norm(v, (self.width,), self.w, self.b, self.eps)
        return out.to(self.rt.dtype)


@dataclasses.dataclass(frozen=True)
class ToyNormConfig:
    vocab_size: int
    hidden_size: int
    n_layers: int
    architecture: str = "ToyNormForCausalLM"


def _toy_norm_kinds(i):
    """(mixer norm, feed-forward norm) of layer i: every neighbourhood of the two kinds of norm in four layers."""
    return (("rmsnorm", "toy_layernorm"), ("toy_layernorm", "rmsnorm"), ("rmsnorm", "rmsnorm"), ("toy_layernorm", "toy_layernorm"))[i % 4]


def _toy_norm_spec(cfg, **kw):
    models = importlib.import_module("daisi-llogos_amd.models")
    rot = P.Rotary(16, 16, 1e4)
    layers = []
    for i in range(cfg.n_layers):
        p = f"layers.{i}."
        kinds = _toy_norm_kinds(i)
        layers.append(models.LayerSpec(
            mixer=("attention", dict(prefix=p + "attn.", hidden=cfg.hidden_size, n_heads=4, n_kv_heads=2, head_dim=16, position=rot)),
            ffn=("swiglu", dict(prefix=p + "ffn.", hidden=cfg.hidden_size, intermediate=48)),
            mixer_norm=(kinds[0], dict(name=p + "n1", width=cfg.hidden_size, eps=1e-5)),
            ffn_norm=(kinds[1], dict(name=p + "n2", width=cfg.hidden_size, eps=1e-5))))
    return models.ModelSpec(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, embed_name="embed.weight",
                            layers=layers, final_norm=("toy_layernorm", dict(name="norm", width=cfg.hidden_size, eps=1e-5)),
                            head_name="head", tie_head=False)


L.register_architecture("ToyNormForCausalLM",
                        lambda d: ToyNormConfig(d["vocab_size"], d["hidden_size"], d["n_layers"]), _toy_norm_spec)


def _plain_toy_norm(w, tokens, n_layers):
    def norm(kind, x, name):
        if kind == "rmsnorm":
            return pm.rms_norm(x, w[name + ".weight"], 1e-5)
        c = x - x.mean(1, keepdims=True)
        return c / np.sqrt((c * c).mean(1, keepdims=True) + 1e-5) * w[name + ".weight"] + w[name + ".bias"]
    T = len(tokens)
    x = pm.embedding(w["embed.weight"], tokens)
    f = pm.rope_frequencies(16, 1e4)
    for i in range(n_layers):
        p = f"layers.{i}."
        kinds = _toy_norm_kinds(i)
        n = norm(kinds[0], x, p + "n1")
        q = pm.rope_split_half(pm.linear(n, w[p + "attn.q_proj.weight"]), range(T), 4, 16, f)
        k = pm.rope_split_half(pm.linear(n, w[p + "attn.k_proj.weight"]), range(T), 2, 16, f)
        x = x + pm.linear(pm.attention(q, k, pm.linear(n, w[p + "attn.v_proj.weight"]), 4, 2, 16), w[p + "attn.o_proj.weight"])
        n = norm(kinds[1], x, p + "n2")
        x = x + pm.swiglu_mlp(n, w[p + "ffn.gate_proj.weight"], w[p + "ffn.up_proj.weight"], w[p + "ffn.down_proj.weight"])
    return pm.linear(norm("toy_layernorm", x, "norm"), w["head.weight"])


@pytest.mark.parametrize("dtype", H.DTYPES)
def test_a_toy_norm_beside_the_products_that_add_themselves_to_the_stream(tmp_path, dtype, monkeypatch):
    """A norm of another form, registered here and written against the plain interface, stands before, between and
    after the built-in parts in every neighbourhood: a product hands its sum to such a norm as a tensor, as
    before, and adds itself to the stream only where an rmsnorm reads next.  Prompts and single tokens against
    the plain model; in bfloat16 the single-token steps do use the one-pass product where they may."""
    from safetensors.torch import load_file
    cfg = {"architectures": ["ToyNormForCausalLM"], "vocab_size": 90, "hidden_size": 64, "n_layers": 5,
           "torch_dtype": "float32"}
    folder = L.write_random_model(str(tmp_path / "toy"), cfg, seed=4)
    w = {k: v.double().numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    eng = L.Engine.from_folder(folder, dtype=dtype, max_tokens=1024, n_slots=3, use_graphs=False)
    calls = []
    real = K.gemm_residual_bf16
    monkeypatch.setattr(K, "gemm_residual_bf16", lambda *a, **kw: (calls.append(a[1].shape), real(*a, **kw))[1])
    rng = np.random.default_rng(3)
    seqs = [rng.integers(0, 90, size=n).tolist() for n in (33, 150, 9)]
    want = [_plain_toy_norm(w, s, 5) for s in seqs]
    tol = 1e-4 if dtype == "float32" else 3e-2
    slots = [eng.alloc_slot() for _ in seqs]
    out = _np(eng.step([(sl, s[:-2]) for sl, s in zip(slots, seqs)], want="last"))
    for i, s in enumerate(seqs):
        assert np.abs(out[i] - want[i][len(s) - 3]).max() <= tol * max(1.0, np.abs(want[i]).max())
    assert not calls                                                     # prompts: more than 16 rows
    for j in (2, 1):
        out = _np(eng.step([(sl, [s[-j]]) for sl, s in zip(slots, seqs)], want="last"))
        for i, s in enumerate(seqs):
            assert np.abs(out[i] - want[i][len(s) - j]).max() <= tol * max(1.0, np.abs(want[i]).max())
    # layers 0..4 have (rms, toy), (toy, rms), (rms, rms), (toy, toy), (rms, toy) and the final norm is a toy: the
    # one-pass product closes a part only where an rmsnorm reads next: o of layers 1 and 2, down of layers 1 and 3
    assert len(calls) == (2 * 4 if dtype == "bfloat16" else 0)


@P.register_feed_forward("toy_routed")
class ToyRoutedFeedForward(P.FeedForward):
    """A router picks one of `n_experts` SwiGLU experts for each token; the expert's output is
    scaled by the router's probability of it.  The routing is decided on the host (tokens are
    gathered per expert), so steps with it are not captured."""

    def __init__(self, prefix: str, hidden: int, intermediate: int, n_experts: int):
        self.router = P.Linear([prefix + "router"], hidden, [n_experts])
        self.experts = [P.SwiGLU(f"{prefix}experts.{e}.", hidden, intermediate) for e in range(n_experts)]

    def tensor_specs(self):
        return self.router.tensor_specs() + [s for e in self.experts for s in e.tensor_specs()]

    def bind(self, get, rt):
        super().bind(get, rt)
        self.router.bind(get, rt)
        for e in self.experts:
            e.bind(get, rt)

    def forward(self, ctx, h):
        logits = self.router.forward(h, out_dtype=torch.float32)            # router logits in 32-bit
        prob = torch.softmax(logits, dim=-1)
        choice = torch.argmax(logits, dim=-1)
        out = torch.zeros((h.shape[0], h.shape[1]), dtype=torch.float32, device=h.device)
        for e, expert in enumerate(self.experts):
            rows = torch.nonzero(choice == e).flatten()
            if rows.numel():
                y = K.sum_parts(expert.forward(ctx, h[rows].contiguous()), None, torch.float32)
                out[rows] = y * prob[rows, e:e + 1]
        return out


@P.register_position("toy_restarting")
class RestartingRotary(P.Rotary):
    """Rotary angles of position modulo `period`: another encoding behind the same interface."""

    def __init__(self, head_dim: int, theta: float, period: int):
        super().__init__(head_dim, head_dim, theta)
        self.period = period

    def prepare(self, ctx):
        key = ("toy_restarting", id(self))
        if key not in ctx.shared:
            ctx.shared[key] = K.rope_table(torch.remainder(ctx.tok_pos, self.period).to(torch.int32), self.inv_freq)
        return ctx.shared[key]


@dataclasses.dataclass(frozen=True)
class RoutedConfig:
    vocab_size: int
    hidden_size: int
    n_layers: int


def _routed_spec(cfg, **kw):
    models = importlib.import_module("daisi-llogos_amd.models")
    layers = []
    for i in range(cfg.n_layers):
        p = f"layers.{i}."
        pos = RestartingRotary(16, 1e4, 8) if i % 2 == 0 else P.Rotary(16, 16, 1e4)
        ffn = ("toy_routed", dict(prefix=p + "moe.", hidden=cfg.hidden_size, intermediate=24, n_experts=3)) if i != 1 else \
            ("swiglu", dict(prefix=p + "ffn.", hidden=cfg.hidden_size, intermediate=56))
        layers.append(models.LayerSpec(
            mixer=("attention", dict(prefix=p + "attn.", hidden=cfg.hidden_size, n_heads=4, n_kv_heads=2, head_dim=16,
                                     position=pos)),
            ffn=ffn,
            mixer_norm=("rmsnorm", dict(name=p + "n1", width=cfg.hidden_size, eps=1e-6)),
            ffn_norm=("rmsnorm", dict(name=p + "n2", width=cfg.hidden_size, eps=1e-6))))
    return models.ModelSpec(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, embed_name="embed.weight",
                            layers=layers, final_norm=("rmsnorm", dict(name="norm", width=cfg.hidden_size, eps=1e-6)),
                            head_name="head", tie_head=True)


L.register_architecture("ToyRoutedForCausalLM",
                        lambda d: RoutedConfig(d["vocab_size"], d["hidden_size"], d["n_layers"]), _routed_spec)


def _plain_routed(w, tokens, n_layers):
    T = len(tokens)
    x = pm.embedding(w["embed.weight"], tokens)
    f = pm.rope_frequencies(16, 1e4)
    for i in range(n_layers):
        p = f"layers.{i}."
        n = pm.rms_norm(x, w[p + "n1.weight"], 1e-6)
        positions = [t % 8 for t in range(T)] if i % 2 == 0 else list(range(T))
        q = pm.rope_split_half(pm.linear(n, w[p + "attn.q_proj.weight"]), positions, 4, 16, f)
        k = pm.rope_split_half(pm.linear(n, w[p + "attn.k_proj.weight"]), positions, 2, 16, f)
        x = x + pm.linear(pm.attention(q, k, pm.linear(n, w[p + "attn.v_proj.weight"]), 4, 2, 16), w[p + "attn.o_proj.weight"])
        n = pm.rms_norm(x, w[p + "n2.weight"], 1e-6)
        if i == 1:
            x = x + pm.swiglu_mlp(n, w[p + "ffn.gate_proj.weight"], w[p + "ffn.up_proj.weight"], w[p + "ffn.down_proj.weight"])
            continue
        logits = pm.linear(n, w[p + "moe.router.weight"])
        prob = pm.softmax(logits)
        d = np.zeros_like(x)
        for t in range(T):
            e = int(np.argmax(logits[t]))
            q_ = f"{p}moe.experts.{e}."
            d[t] = prob[t, e] * pm.swiglu_mlp(n[t:t + 1], w[q_ + "gate_proj.weight"], w[q_ + "up_proj.weight"], w[q_ + "down_proj.weight"])[0]
        x = x + d
    return pm.linear(pm.rms_norm(x, w["norm.weight"], 1e-6), w["embed.weight"])


def test_a_toy_feed_forward_with_routing_and_another_position_encoding(tmp_path):
    """Registered here, built from a model description and stepped by the engine, whole and in
    an unequal batch followed by single tokens, without a change to the library's files; a model
    with a part that cannot be captured runs its single-token steps kernel by kernel."""
    from safetensors.torch import load_file
    cfg = {"architectures": ["ToyRoutedForCausalLM"], "vocab_size": 70, "hidden_size": 48, "n_layers": 3,
           "torch_dtype": "float32"}
    folder = L.write_random_model(str(tmp_path / "routed"), cfg, seed=4)
    w = {k: v.double().numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    # spread the router's logits so that the experts in use differ from token to token
    assert sorted(k for k in w if "router" in k) == ["layers.0.moe.router.weight", "layers.2.moe.router.weight"]
    eng = L.Engine.from_folder(folder, dtype="float32", max_tokens=512, n_slots=3)
    assert eng.graphs is None                                           # the routed part decides on the host
    rng = np.random.default_rng(1)
    seqs = [rng.integers(0, 70, size=n).tolist() for n in (40, 9, 21)]
    want = [_plain_routed(w, s, 3) for s in seqs]
    used = {int(np.argmax(pm.linear(pm.rms_norm(pm.embedding(w["embed.weight"], s), w["layers.0.n2.weight"], 1e-6),
                                    w["layers.0.moe.router.weight"])[t])) for s in seqs for t in range(len(s))}
    assert len(used) >= 2                                               # more than one expert is in play
    slot = eng.alloc_slot()
    H.close(_np(eng.step([(slot, seqs[0])], want="all")), want[0], "float32", "routed whole")
    eng.free_slot(slot)
    slots = [eng.alloc_slot() for _ in seqs]
    cut = [30, 4, 20]
    out = _np(eng.step([(sl, s[:c]) for sl, s, c in zip(slots, seqs, cut)], want="all"))
    H.close(out, np.concatenate([wnt[:c] for wnt, c in zip(want, cut)]), "float32", "routed unequal batch")
    for t in range(5):
        live = [i for i in range(3) if cut[i] + t < len(seqs[i])]
        out = _np(eng.step([(slots[i], [seqs[i][cut[i] + t]]) for i in live], want="last"))
        H.close(out, np.stack([want[i][cut[i] + t] for i in live]), "float32", f"routed token {t}")


# ---------------------------------------------------------------------------
# a toy block with two mixers side by side, a scaled embedding and capped logits, defined here
# ---------------------------------------------------------------------------
@P.register_block("toy_two_mixers")
class TwoMixers(P.Block):
    """x += pending; h = norm(x); x += mixer_0(h) + mixer_1(h); pending = ffn(ffn_norm(x)).
    Each mixer has a cache of its own (keys and values for the one, fixed-size state for the other)."""

    def __init__(self, norm, mixers, ffn_norm, ffn):
        self.norm, self._mixers, self.ffn_norm, self.ffn = norm, list(mixers), ffn_norm, ffn

    def mixers(self):
        return self._mixers

    def feed_forwards(self):
        return [self.ffn]

    def parts(self):
        return [self.norm, *self._mixers, self.ffn_norm, self.ffn]

    def forward(self, ctx, x, pending, caches):
        h = self.norm.forward(x, pending)
        a = self._mixers[0].forward(ctx, h, caches[0])
        K.residual_add(x, K.sum_parts(a, None, torch.float32))
        b = self._mixers[1].forward(ctx, h, caches[1])
        return x, self.ffn.forward(ctx, self.ffn_norm.forward(x, b))


@dataclasses.dataclass(frozen=True)
class TwoMixerConfig:
    vocab_size: int
    hidden_size: int
    n_layers: int


def _two_mixer_spec(cfg, **kw):
    models = importlib.import_module("daisi-llogos_amd.models")
    rot = P.Rotary(16, 16, 1e4)
    norm = lambda name: ("norm", "rmsnorm", dict(name=name, width=cfg.hidden_size, eps=1e-6))
    layers = []
    for i in range(cfg.n_layers):
        p = f"layers.{i}."
        layers.append(models.LayerSpec(block="toy_two_mixers", more={
            "norm": norm(p + "n1"),
            "mixers": [("mixer", "attention", dict(prefix=p + "attn.", hidden=cfg.hidden_size, n_heads=2, n_kv_heads=1,
                                                   head_dim=16, position=rot)),
                       ("mixer", "toy_running_mean", dict(prefix=p, hidden=cfg.hidden_size))],
            "ffn_norm": norm(p + "n2"),
            "ffn": ("feed_forward", "swiglu", dict(prefix=p + "ffn.", hidden=cfg.hidden_size, intermediate=56))}))
    return models.ModelSpec(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, embed_name="embed.weight",
                            layers=layers, final_norm=("rmsnorm", dict(name="norm", width=cfg.hidden_size, eps=1e-6)),
                            head_name="head", tie_head=False, embed_scale=3.0, logit_scale=0.5, logit_softcap=2.0)


L.register_architecture("ToyTwoMixersForCausalLM",
                        lambda d: TwoMixerConfig(d["vocab_size"], d["hidden_size"], d["n_layers"]), _two_mixer_spec)


def _plain_two_mixers(w, tokens, n_layers):
    T = len(tokens)
    x = 3.0 * pm.embedding(w["embed.weight"], tokens)
    f = pm.rope_frequencies(16, 1e4)
    for i in range(n_layers):
        p = f"layers.{i}."
        n = pm.rms_norm(x, w[p + "n1.weight"], 1e-6)
        q = pm.rope_split_half(pm.linear(n, w[p + "attn.q_proj.weight"]), range(T), 2, 16, f)
        k = pm.rope_split_half(pm.linear(n, w[p + "attn.k_proj.weight"]), range(T), 1, 16, f)
        a = pm.linear(pm.attention(q, k, pm.linear(n, w[p + "attn.v_proj.weight"]), 2, 1, 16), w[p + "attn.o_proj.weight"])
        b = pm.linear(np.cumsum(n, axis=0) / np.arange(1, T + 1)[:, None], w[p + "mix.weight"])
        x = x + a + b
        n = pm.rms_norm(x, w[p + "n2.weight"], 1e-6)
        x = x + pm.swiglu_mlp(n, w[p + "ffn.gate_proj.weight"], w[p + "ffn.up_proj.weight"], w[p + "ffn.down_proj.weight"])
    logits = 0.5 * pm.linear(pm.rms_norm(x, w["norm.weight"], 1e-6), w["head.weight"])
    return 2.0 * np.tanh(logits / 2.0)


def test_a_toy_block_with_two_mixers_and_scaled_embedding_and_logits(tmp_path):
    """A block that holds two mixers (attention with keys and values, a running mean with
    fixed-size state), an embedding scale and scaled, capped logits: registered here, built
    from a model description and stepped whole, in an unequal batch and token by token."""
    from safetensors.torch import load_file
    cfg = {"architectures": ["ToyTwoMixersForCausalLM"], "vocab_size": 80, "hidden_size": 40, "n_layers": 2,
           "torch_dtype": "float32"}
    folder = L.write_random_model(str(tmp_path / "two"), cfg, seed=6)
    w = {k: v.double().numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    w["head.weight"] *= 40.0                                            # logits large enough for the cap to bend them
    eng = L.Engine.from_folder(folder, dtype="float32", max_tokens=512, n_slots=3)
    eng.model.head.weight.mul_(40.0)
    needs = eng.model.cache_needs()
    assert [(kv is not None, st is not None) for kv, st in needs] == [(True, False), (False, True)] * 2
    assert eng.model.entry_units == [[0, 1], [2, 3]] and eng.graphs is None      # the running mean reads host lists
    rng = np.random.default_rng(2)
    seqs = [rng.integers(0, 80, size=n).tolist() for n in (70, 5, 33)]
    want = [_plain_two_mixers(w, s, 2) for s in seqs]
    assert np.abs(want[0]).max() > 1.5 and np.abs(want[0]).max() < 2.0          # the cap is at work
    slot = eng.alloc_slot()
    H.close(_np(eng.step([(slot, seqs[0])], want="all")), want[0], "float32", "two mixers whole")
    eng.free_slot(slot)
    slots = [eng.alloc_slot() for _ in seqs]
    cut = [66, 2, 30]
    out = _np(eng.step([(sl, s[:c]) for sl, s, c in zip(slots, seqs, cut)], want="all"))
    H.close(out, np.concatenate([wnt[:c] for wnt, c in zip(want, cut)]), "float32", "two mixers, unequal batch")
    for t in range(3):
        out = _np(eng.step([(slots[i], [seqs[i][cut[i] + t]]) for i in range(3)], want="last"))
        H.close(out, np.stack([want[i][cut[i] + t] for i in range(3)]), "float32", f"two mixers, token {t}")


# ---------------------------------------------------------------------------
# a toy mixer with state whose single-token steps are captured and replayed
# ---------------------------------------------------------------------------
@P.register_mixer("toy_running_mean_on_device")
class RunningMeanOnDevice(P.Mixer):
    """out_t = g * mean(h_0 .. h_t) with a weight vector g; single-token steps read and write
    the state through the step's device tensors alone, so they may be captured."""
    graph_safe = True

    def __init__(self, prefix, hidden):
        self.prefix, self.hidden = prefix, hidden

    def tensor_specs(self):
        return [P.TensorSpec(self.prefix + "gain.weight", (self.hidden,), "norm")]

    def state_spec(self):
        return P.StateSpec((self.hidden,), torch.float32)

    def bind(self, get, rt):
        self.rt = rt
        self.g = get(self.prefix + "gain.weight").to(device=rt.device, dtype=torch.float32)

    def forward(self, ctx, h, cache):
        if ctx.is_decode:
            slots = ctx.slots.long()
            run = cache.state.index_select(0, slots) + h.float()
            cache.state.index_copy_(0, slots, run)
            return (run / (ctx.tok_pos + 1).float()[:, None] * self.g).to(h.dtype)
        out = torch.empty_like(h)
        for b in range(ctx.batch):
            lo, hi = ctx.cu_seqlens[b], ctx.cu_seqlens[b + 1]
            run = torch.cumsum(h[lo:hi].float(), 0) + cache.state[ctx.slot_ids[b]]
            cache.state[ctx.slot_ids[b]] = run[-1]
            count = torch.arange(ctx.starts[b] + 1, ctx.starts[b] + hi - lo + 1, device=h.device)[:, None]
            out[lo:hi] = (run / count * self.g).to(h.dtype)
        return out


def _state_graph_spec(cfg, **kw):
    models = importlib.import_module("daisi-llogos_amd.models")
    layers = []
    for i in range(cfg.n_layers):
        p = f"layers.{i}."
        layers.append(models.LayerSpec(
            mixer=("toy_running_mean_on_device", dict(prefix=p, hidden=cfg.hidden_size)),
            ffn=("swiglu", dict(prefix=p + "ffn.", hidden=cfg.hidden_size, intermediate=56)),
            mixer_norm=("rmsnorm", dict(name=p + "n1", width=cfg.hidden_size, eps=1e-6)),
            ffn_norm=("rmsnorm", dict(name=p + "n2", width=cfg.hidden_size, eps=1e-6))))
    return models.ModelSpec(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, embed_name="embed.weight",
                            layers=layers, final_norm=("rmsnorm", dict(name="norm", width=cfg.hidden_size, eps=1e-6)),
                            head_name="head", tie_head=False)


L.register_architecture("ToyStateOnDeviceForCausalLM",
                        lambda d: ToyConfig(d["vocab_size"], d["hidden_size"], d["n_layers"]), _state_graph_spec)


def test_captured_steps_of_a_mixer_with_state_advance_the_state_once(tmp_path):
    """A captured step is run once for real before its capture and then replayed: fixed-size
    state must come out advanced once, not twice.  Replayed steps against the same steps launched
    kernel by kernel, bit for bit, through several batch sizes (each a new capture), and against
    the plain running mean."""
    from safetensors.torch import load_file
    cfg = {"architectures": ["ToyStateOnDeviceForCausalLM"], "vocab_size": 60, "hidden_size": 40, "n_layers": 2,
           "torch_dtype": "float32"}
    folder = L.write_random_model(str(tmp_path / "state"), cfg, seed=9)
    w = {k: v.double().numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}

    def plain(tokens):
        x = pm.embedding(w["embed.weight"], tokens)
        for i in range(2):
            p = f"layers.{i}."
            n = pm.rms_norm(x, w[p + "n1.weight"], 1e-6)
            x = x + np.cumsum(n, axis=0) / np.arange(1, len(tokens) + 1)[:, None] * w[p + "gain.weight"]
            n = pm.rms_norm(x, w[p + "n2.weight"], 1e-6)
            x = x + pm.swiglu_mlp(n, w[p + "ffn.gate_proj.weight"], w[p + "ffn.up_proj.weight"], w[p + "ffn.down_proj.weight"])
        return pm.linear(pm.rms_norm(x, w["norm.weight"], 1e-6), w["head.weight"])

    engines = [L.Engine.from_folder(folder, dtype="float32", max_tokens=512, n_slots=4, use_graphs=g) for g in (True, False)]
    assert engines[0].graphs is not None and engines[1].graphs is None
    rng = np.random.default_rng(4)
    seqs = [rng.integers(0, 60, size=n).tolist() for n in (30, 12, 25)]
    want = [plain(s) for s in seqs]
    cut = [9, 2, 5]
    slots = [[e.alloc_slot() for _ in seqs] for e in engines]
    for e, sl in zip(engines, slots):
        e.step([(s, q[:c]) for s, q, c in zip(sl, seqs, cut)], want=None)
    for t in range(10):
        live = [i for i in range(3) if cut[i] + t < len(seqs[i]) and (i != 1 or t < 4)]     # the batch shrinks: 3, then 2
        outs = [_np(e.step([(sl[i], [seqs[i][cut[i] + t]]) for i in live], want="last")) for e, sl in zip(engines, slots)]
        assert np.array_equal(outs[0], outs[1]), f"token {t}: replayed and launched steps differ by {np.abs(outs[0] - outs[1]).max()}"
        H.close(outs[0], np.stack([want[i][cut[i] + t] for i in live]), "float32", f"state on device, token {t}")
    assert len(engines[0].graphs.graphs) == 2


def test_a_slot_beyond_the_first_count_between_replays_of_a_captured_step(tmp_path):
    """The cache starts with two slots.  Two sequences are stepped through captured graphs; then a
    third sequence takes a slot the cache did not have, which makes the per-slot state tensors
    anew (the captured graphs hold the old ones' addresses and must be dropped), and all three go
    on.  Replayed steps against launched ones bit for bit, and against the plain running mean: a
    graph that still wrote the old state tensor, or a state that did not move with its slot,
    would show at the first token after the growth."""
    from safetensors.torch import load_file
    cfg = {"architectures": ["ToyStateOnDeviceForCausalLM"], "vocab_size": 60, "hidden_size": 40, "n_layers": 2,
           "torch_dtype": "float32"}
    folder = L.write_random_model(str(tmp_path / "grow"), cfg, seed=12)
    w = {k: v.double().numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}

    def plain(tokens):
        x = pm.embedding(w["embed.weight"], tokens)
        for i in range(2):
            p = f"layers.{i}."
            n = pm.rms_norm(x, w[p + "n1.weight"], 1e-6)
            x = x + np.cumsum(n, axis=0) / np.arange(1, len(tokens) + 1)[:, None] * w[p + "gain.weight"]
            n = pm.rms_norm(x, w[p + "n2.weight"], 1e-6)
            x = x + pm.swiglu_mlp(n, w[p + "ffn.gate_proj.weight"], w[p + "ffn.up_proj.weight"], w[p + "ffn.down_proj.weight"])
        return pm.linear(pm.rms_norm(x, w["norm.weight"], 1e-6), w["head.weight"])

    engines = [L.Engine.from_folder(folder, dtype="float32", max_tokens=512, n_slots=2, use_graphs=g) for g in (True, False)]
    rng = np.random.default_rng(6)
    seqs = [rng.integers(0, 60, size=n).tolist() for n in (24, 20, 18)]
    want = [plain(s) for s in seqs]
    cut = [7, 3, 5]
    slots = [[e.alloc_slot() for _ in range(2)] for e in engines]
    for e, sl in zip(engines, slots):
        e.step([(s, q[:c]) for s, q, c in zip(sl, seqs, cut)], want=None)
    fed = list(cut)

    def one_token_each(live, what):
        outs = [_np(e.step([(sl[i], [seqs[i][fed[i]]]) for i in live], want="last")) for e, sl in zip(engines, slots)]
        assert np.array_equal(outs[0], outs[1]), f"{what}: replayed and launched steps differ by {np.abs(outs[0] - outs[1]).max()}"
        H.close(outs[0], np.stack([want[i][fed[i]] for i in live]), "float32", what)
        for i in live:
            fed[i] += 1

    for t in range(4):
        one_token_each([0, 1], f"two sequences, token {t}")
    held = engines[0].cache.states[0]
    assert engines[0].cache.slots.n_slots == 2 and len(engines[0].graphs.graphs) == 1
    for e, sl in zip(engines, slots):
        sl.append(e.alloc_slot())                                           # the third slot: the cache grows
        e.step([(sl[2], seqs[2][:cut[2]])], want=None)
    assert engines[0].cache.slots.n_slots > 2 and engines[0].cache.states[0] is not held
    for t in range(6):
        one_token_each([0, 1, 2], f"three sequences after the growth, token {t}")
    one_token_each([2, 0], "two of them, in another order")
    assert set(engines[0].graphs.graphs) == {(3, ()), (2, ())}             # the graphs of before the growth are gone


# ---------------------------------------------------------------------------
# a toy mixer with keys and values in the cache and a position scheme that is no rotation, defined here
# ---------------------------------------------------------------------------
@P.register_mixer("toy_distance_bias_attention")
class DistanceBiasAttention(P.Mixer):
    """Attention without rotation: the score of query i and key j is q . k / sqrt(hd) - slope_h (i - j).
    It keeps its keys and values in the cache's pages, which it reaches through the cache's own
    rule for where a (token, dimension) lies in a page (cache/pages.py), with plain tensor
    operations: nothing of the framework knows of it."""

    def __init__(self, prefix, hidden, n_heads, head_dim, slopes):
        self.prefix, self.hidden, self.nh, self.hd, self.slopes = prefix, hidden, n_heads, head_dim, list(slopes)

    def tensor_specs(self):
        return [P.TensorSpec(self.prefix + n + ".weight", shape, "matrix")
                for n, shape in (("q", (self.nh * self.hd, self.hidden)), ("k", (self.nh * self.hd, self.hidden)),
                                 ("v", (self.nh * self.hd, self.hidden)), ("o", (self.hidden, self.nh * self.hd)))]

    def kv_spec(self):
        return P.KVSpec(self.nh, self.hd)

    def bind(self, get, rt):
        pages = importlib.import_module("daisi-llogos_amd.cache.pages")
        self.rt = rt
        self.w = {n: get(self.prefix + n + ".weight").to(device=rt.device, dtype=torch.float32) for n in "qkvo"}
        ki, vi = pages.page_offsets(self.hd)
        self.ki, self.vi = torch.tensor(ki, device=rt.device), torch.tensor(vi, device=rt.device)     # [64, hd]

    def forward(self, ctx, h, cache):
        nh, hd = self.nh, self.hd
        x = h.float()
        q, k, v = (x @ self.w[n].T for n in "qkv")
        out = torch.empty((h.shape[0], nh * hd), dtype=torch.float32, device=h.device)
        slopes = torch.tensor(self.slopes, device=h.device)[:, None, None]
        for b in range(ctx.batch):
            lo, hi = ctx.cu_seqlens[b], ctx.cu_seqlens[b + 1]
            start, n = ctx.starts[b], ctx.cu_seqlens[b + 1] - ctx.cu_seqlens[b]
            pos = torch.arange(start, start + n, device=h.device)
            page, at = cache.table[b].long()[pos // 64], pos % 64
            for pool, rule, rows in ((cache.k_pool, self.ki, k), (cache.v_pool, self.vi, v)):
                flat = pool.view(pool.shape[0], nh, 64 * hd)
                new = rows[lo:hi].view(n, nh, hd).to(pool.dtype)
                flat[page[:, None, None], torch.arange(nh, device=h.device)[None, :, None], rule[at][:, None, :]] = new
            every = torch.arange(0, start + n, device=h.device)                        # all positions so far, from the pages
            page, at = cache.table[b].long()[every // 64], every % 64
            heads = torch.arange(nh, device=h.device)[None, :, None]
            keys = cache.k_pool[page[:, None, None], heads, self.ki[at][:, None, :]].float()      # [positions, heads, hd]
            vals = cache.v_pool[page[:, None, None], heads, self.vi[at][:, None, :]].float()
            s = torch.einsum("ihd,jhd->hij", q[lo:hi].view(n, nh, hd), keys) / hd ** 0.5
            dist = (pos[:, None] - every[None, :]).float()
            s = (s - slopes * dist).masked_fill(dist[None] < 0, float("-inf"))
            out[lo:hi] = torch.einsum("hij,jhd->ihd", torch.softmax(s, -1), vals).reshape(n, nh * hd)
        return (out @ self.w["o"].T).to(h.dtype)


def _bias_spec(cfg, **kw):
    models = importlib.import_module("daisi-llogos_amd.models")
    layers = []
    for i in range(cfg.n_layers):
        p = f"layers.{i}."
        layers.append(models.LayerSpec(
            mixer=("toy_distance_bias_attention", dict(prefix=p + "mix.", hidden=cfg.hidden_size, n_heads=3, head_dim=16,
                                                       slopes=[0.5, 0.125, 0.03125])),
            ffn=("swiglu", dict(prefix=p + "ffn.", hidden=cfg.hidden_size, intermediate=56)),
            mixer_norm=("rmsnorm", dict(name=p + "n1", width=cfg.hidden_size, eps=1e-6)),
            ffn_norm=("rmsnorm", dict(name=p + "n2", width=cfg.hidden_size, eps=1e-6))))
    return models.ModelSpec(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, embed_name="embed.weight",
                            layers=layers, final_norm=("rmsnorm", dict(name="norm", width=cfg.hidden_size, eps=1e-6)),
                            head_name="head", tie_head=False)


L.register_architecture("ToyDistanceBiasForCausalLM",
                        lambda d: ToyConfig(d["vocab_size"], d["hidden_size"], d["n_layers"]), _bias_spec)


def test_a_toy_mixer_with_cached_keys_and_a_position_scheme_of_its_own(tmp_path):
    """A mixer whose positions enter as a bias on the scores (no rotation, no table of angles) and
    whose keys and values live in the cache's pages is registered, built and stepped from here:
    whole prompts, then token by token in a batch of unequal lengths across a page's end, with
    slots and pages used again, against plain arithmetic."""
    from safetensors.torch import load_file
    cfg = {"architectures": ["ToyDistanceBiasForCausalLM"], "vocab_size": 70, "hidden_size": 40, "n_layers": 2,
           "torch_dtype": "float32"}
    folder = L.write_random_model(str(tmp_path / "bias"), cfg, seed=6)
    w = {k: v.double().numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    slopes = np.array([0.5, 0.125, 0.03125])

    def plain(tokens):
        T = len(tokens)
        x = pm.embedding(w["embed.weight"], tokens)
        dist = np.arange(T)[:, None] - np.arange(T)[None, :]
        for i in range(2):
            p = f"layers.{i}."
            n = pm.rms_norm(x, w[p + "n1.weight"], 1e-6)
            q, k, v = (pm.linear(n, w[p + f"mix.{m}.weight"]).reshape(T, 3, 16) for m in "qkv")
            a = np.zeros((T, 3, 16))
            for hh in range(3):
                s = q[:, hh] @ k[:, hh].T / 4.0 - slopes[hh] * dist
                s = np.where(dist < 0, -np.inf, s)
                a[:, hh] = np.stack([pm.softmax(r) for r in s]) @ v[:, hh]
            x = x + pm.linear(a.reshape(T, 48), w[p + "mix.o.weight"])
            n = pm.rms_norm(x, w[p + "n2.weight"], 1e-6)
            x = x + pm.swiglu_mlp(n, w[p + "ffn.gate_proj.weight"], w[p + "ffn.up_proj.weight"], w[p + "ffn.down_proj.weight"])
        return pm.linear(pm.rms_norm(x, w["norm.weight"], 1e-6), w["head.weight"])

    eng = L.Engine.from_folder(folder, dtype="float32", max_tokens=64 * 5, n_slots=3)
    assert all(kv == P.KVSpec(3, 16) and st is None for kv, st in eng.model.cache_needs())
    assert eng.graphs is None or not eng.model.graph_safe                 # the mixer reads the step on the host: never captured
    rng = np.random.default_rng(1)
    seqs = [rng.integers(0, 70, size=n).tolist() for n in (75, 9, 130)]
    want = [plain(s) for s in seqs]
    for s, wnt in zip(seqs[:2], want):
        slot = eng.alloc_slot()
        H.close(_np(eng.step([(slot, s)], want="all")), wnt, "float32", "distance bias, whole")
        eng.free_slot(slot)
    slots = [eng.alloc_slot() for _ in seqs]
    cut = [60, 3, 120]
    out = _np(eng.step([(sl, s[:c]) for sl, s, c in zip(slots, seqs, cut)], want="last"))
    H.close(out, np.stack([wnt[c - 1] for wnt, c in zip(want, cut)]), "float32", "distance bias, prompts")
    for t in range(10):                                                   # across the ends of pages at 64 and 128
        live = [i for i in range(3) if cut[i] + t < len(seqs[i])]
        got = _np(eng.step([(slots[i], [seqs[i][cut[i] + t]]) for i in live], want="last"))
        H.close(got, np.stack([want[i][cut[i] + t] for i in live]), "float32", f"distance bias, token {t}")
        for i in live:
            if cut[i] + t + 1 == len(seqs[i]):
                eng.free_slot(slots[i])
