"""Each part alone on the GPU against the plain implementation's function of the same
name, in float32 and bfloat16; and a toy mixer with a state of its own, defined here,
registered, built into a model through the registries and stepped through the engine
without a change to the framework's files; likewise a feed-forward with routing, a position
encoding with parameters and a mixer that keeps no cache."""

from dataclasses import dataclass
from typing import ClassVar

import pytest
import torch

import plain_model as pm
from helpers import gpu_ops
from atom_amd.cache import CacheKind, CacheManager, GroupSpec, kind_of, register_cache_kind, unregister_cache_kind
from atom_amd.config import ModelConfig, register_architecture, unregister_architecture
from atom_amd.engine.context import BatchView, KVBinding, StepContext
from atom_amd.engine.core import StepEntry, build_core, load_model
from atom_amd.models.model import ModelSpec
from atom_amd.parts import (FEED_FORWARDS, MIXERS, POSITION_ENCODINGS, FeedForward, GatedMLP,
                            GroupedQueryAttention, LMHead, Mixer, ParamSpec, PartChoice, PositionEncoding, PreNormBlock,
                            RMSNorm, RotaryEncoding, StateNeed, TokenEmbedding)
from atom_amd.weights import write_random_model

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]
TOL = {torch.float32: 1e-5, torch.bfloat16: 2.5e-2}


def rnd(shape, seed, scale=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale


def fill(part, dtype, seed=0, scale=0.3):
    """Random parameters for a part and its children; returns them by full name in float64."""
    out = {}
    for k, p in enumerate(part.walk()):
        for local, spec in p.param_specs().items():
            value = rnd(spec.shape, seed * 1000 + k * 10 + len(out), scale)
            if spec.init == "one_plus_normal":
                value = 1 + value
            target = torch.float32 if spec.kind == "vector" else dtype
            p.params[local] = value.to(target).to(DEV)
            out[p.full_name(local)] = p.params[local].double().cpu()
        p.finalize(torch.device(DEV), dtype)
    return out


def ctx_for(dtype, positions, page_size=16, group=0, num_pages=None, mixer=None):
    """A one-request step context: the request's tokens at ``positions`` (consecutive), with what
    ``mixer`` asks for in its ``prepare_step``."""
    n = len(positions)
    end = positions[-1] + 1
    num_pages = num_pages or -(-end // page_size) + 2
    mgr = CacheManager([GroupSpec(page_size, num_pages)], 1)
    mgr.open("r")
    mgr.cover("r", 0, end)
    table = torch.tensor([mgr.block_table("r", 0)], dtype=torch.int32, device=DEV)
    pos = torch.tensor(positions, dtype=torch.int32, device=DEV)
    slots = torch.from_numpy(mgr.slot_mapping("r", 0, positions[0], n)).to(DEV)
    i32 = lambda values: torch.tensor(values, dtype=torch.int32, device=DEV)  # noqa: E731
    ctx = StepContext(ops=gpu_ops(), dtype=dtype, device=torch.device(DEV), num_tokens=n, num_seqs=1, positions=pos,
                      token_seq=torch.zeros(n, dtype=torch.int32, device=DEV), cu_seqlens_q=i32([0, n]),
                      context_lens=i32([end]), cached_lens=i32([positions[0]]), slot_of_seq=i32([0]),
                      block_tables={group: table}, slot_mappings={group: slots}, page_sizes={group: page_size},
                      num_prefill=1 if n > 1 else 0, max_q_len=n, max_context_len=end,
                      seq_starts=[0], seq_lens=[n], seq_cached=[positions[0]], state_slots=[0])
    if mixer is not None:   # what the engine does with a mixer's ``prepare_step``: its arrays, on the device
        view = BatchView(ops=ctx.ops, dtype=dtype, q_lens=[n], cached=[positions[0]], num_prefill=ctx.num_prefill,
                         page_sizes=[page_size])
        ctx.prepared[mixer.step_key()] = {name: torch.from_numpy(a).to(DEV)
                                          for name, a in mixer.prepare_step(view).items()}
    return ctx, num_pages


def check(got, want, dtype):
    got, want = got.double().cpu(), want.double()
    scale = max(1e-6, float(want.abs().max()))
    assert float((got - want).abs().max()) <= TOL[dtype] * scale


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_part(dtype):
    norm = RMSNorm(136, 3e-6, prefix="n")
    w = fill(norm, dtype)["n.weight"]
    ctx, _ = ctx_for(dtype, [0, 1, 2, 3, 4])
    x = rnd((5, 136), 1, 2.0).to(dtype)
    check(norm.forward(ctx, x.to(DEV)), pm.rms_norm(x.double(), w, 3e-6), dtype)
    y, res = norm.forward_residual(ctx, x.to(DEV), None)
    assert res.dtype == torch.float32 and torch.equal(res.cpu(), x.float())
    check(y, pm.rms_norm(x.double(), w, 3e-6), dtype)
    x2 = rnd((5, 136), 2).to(dtype)
    y2, res2 = norm.forward_residual(ctx, x2.to(DEV), res)
    want_y, want_res = pm.add_rms_norm(x2.double(), x.double(), w, 3e-6)
    check(y2, want_y, dtype)
    check(res2, want_res, torch.float32)
    rows = torch.tensor([4, 1], dtype=torch.int32, device=DEV)
    y3 = norm.forward_rows(ctx, x2.to(DEV), res2.clone(), rows)
    want3, _ = pm.add_rms_norm(x2.double()[[4, 1]], res2.double().cpu()[[4, 1]], w, 3e-6)
    check(y3, want3, dtype)


def test_rotary_tables():
    rope = RotaryEncoding(head_dim=64, theta=5e5, max_positions=300)
    rope.finalize(torch.device(DEV), torch.bfloat16)
    cos, sin = pm.rope_angles(torch.arange(300), 64, 5e5)
    assert rope.cos.dtype == torch.float32 and rope.cos.shape == (300, 32)
    assert torch.equal(rope.cos.cpu(), cos) and torch.equal(rope.sin.cpu(), sin)
    with pytest.raises(ValueError):
        RotaryEncoding(head_dim=64, theta=1e4, max_positions=8, rotary_dim=65)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hq,hkv,d,bias,window", [(4, 2, 16, False, None), (6, 3, 32, True, None), (8, 2, 64, True, 9),
                                                  (3, 3, 48, False, None)])
def test_attention_part(dtype, hq, hkv, d, bias, window):
    hidden = 72
    rope = PartChoice("rotary", {"theta": 1e4, "max_positions": 128})
    attn = GroupedQueryAttention(hidden, hq, hkv, d, qkv_bias=bias, qk_norm=True, norm_eps=1e-5, window=window,
                                 position_encoding=rope, prefix="a")
    w = fill(attn, dtype, seed=3, scale=0.2)
    n = 37
    ctx, pages = ctx_for(dtype, list(range(n)), page_size=8, mixer=attn)
    cache = KVBinding(0, torch.zeros((pages, hkv, 8, d), dtype=dtype, device=DEV),
                      torch.zeros((pages, hkv, d, 8), dtype=dtype, device=DEV))
    x = rnd((n, hidden), 4).to(dtype)
    got = attn.forward(ctx, x.to(DEV), cache)
    qkv = w["a.qkv.weight"]
    plain_w = {"q_proj.weight": qkv[:hq * d], "k_proj.weight": qkv[hq * d:(hq + hkv) * d],
               "v_proj.weight": qkv[(hq + hkv) * d:], "o_proj.weight": w["a.o.weight"],
               "q_norm.weight": w["a.q_norm.weight"], "k_norm.weight": w["a.k_norm.weight"]}
    if bias:
        b = w["a.qkv.bias"]
        plain_w.update({"q_proj.bias": b[:hq * d], "k_proj.bias": b[hq * d:(hq + hkv) * d], "v_proj.bias": b[(hq + hkv) * d:]})
    cfg = dict(num_attention_heads=hq, num_key_value_heads=hkv, head_dim=d, rms_norm_eps=1e-5, rope_theta=1e4)
    want, _ = pm.self_attention(x.double(), torch.arange(n), plain_w, cfg, window)
    check(got, want, dtype)
    # the same tokens in two steps over the cache the first step left
    cache2 = KVBinding(0, torch.zeros_like(cache.k_cache), torch.zeros_like(cache.v_cache))
    ctx_a, _ = ctx_for(dtype, list(range(20)), page_size=8, num_pages=pages, mixer=attn)
    ctx_b, _ = ctx_for(dtype, list(range(20, n)), page_size=8, num_pages=pages, mixer=attn)
    first = attn.forward(ctx_a, x[:20].to(DEV), cache2)
    second = attn.forward(ctx_b, x[20:].to(DEV), cache2)
    check(torch.cat((first, second)), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_mlp_part(dtype):
    mlp = GatedMLP(96, 160, prefix="m")
    w = fill(mlp, dtype, seed=5)
    ctx, _ = ctx_for(dtype, [0, 1, 2])
    x = rnd((3, 96), 6).to(dtype)
    gu = w["m.gate_up.weight"]
    want = pm.gated_mlp(x.double(), gu[:160], gu[160:], w["m.down.weight"])
    check(gpu_ops().materialize(mlp.forward(ctx, x.to(DEV))), want, dtype)   # few rows: the down product is still pending
    with pytest.raises(ValueError):
        GatedMLP(8, 8, activation="gelu")


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_and_head(dtype):
    emb = TokenEmbedding(311, 96, prefix="e")
    w = fill(emb, dtype, seed=7)["e.weight"]
    ctx, _ = ctx_for(dtype, [0, 1, 2, 3])
    ids = torch.tensor([310, 0, 17, 17], dtype=torch.int32, device=DEV)
    x = emb.forward(ctx, ids)
    assert x.dtype == dtype and torch.equal(x.double().cpu(), w[[310, 0, 17, 17]])
    tied = LMHead(311, 96, tied_to=emb, prefix="h")
    assert tied.param_specs() == {} and tied.weight is emb.params["weight"]
    logits = tied.forward(ctx, x)
    assert logits.dtype == torch.float32
    check(logits, x.double().cpu() @ w.T, dtype)
    own = LMHead(311, 96, prefix="h")
    hw = fill(own, dtype, seed=8)["h.weight"]
    check(own.forward(ctx, x), x.double().cpu() @ hw.T, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_prenorm_block(dtype):
    norm = PartChoice("rmsnorm", {"size": 64, "eps": 1e-6})
    block = PreNormBlock(
        mixer=PartChoice("attention", {"hidden_size": 64, "num_heads": 4, "num_kv_heads": 2, "head_dim": 16,
                                       "qk_norm": True, "position_encoding": PartChoice("rotary", {"theta": 1e4, "max_positions": 64})}),
        feed_forward=PartChoice("gated_mlp", {"hidden_size": 64, "intermediate_size": 100}), norm=norm, prefix="model.layers.0")
    w = fill(block, dtype, seed=9, scale=0.2)
    n = 21
    ctx, pages = ctx_for(dtype, list(range(n)), mixer=block.mixer)
    cache = KVBinding(0, torch.zeros((pages, 2, 16, 16), dtype=dtype, device=DEV), torch.zeros((pages, 2, 16, 16), dtype=dtype, device=DEV))
    x, r = rnd((n, 64), 10).to(dtype), rnd((n, 64), 11)
    hidden, res = block.forward(ctx, x.to(DEV), r.to(DEV), cache)
    p = "model.layers.0."
    summed = x.double() + r.double()
    h = pm.rms_norm(summed, w[p + "input_layernorm.weight"], 1e-6)
    qkv = w[p + "self_attn.qkv.weight"]
    aw = {"q_proj.weight": qkv[:64], "k_proj.weight": qkv[64:96], "v_proj.weight": qkv[96:],
          "o_proj.weight": w[p + "self_attn.o.weight"], "q_norm.weight": w[p + "self_attn.q_norm.weight"],
          "k_norm.weight": w[p + "self_attn.k_norm.weight"]}
    cfg = dict(num_attention_heads=4, num_key_value_heads=2, head_dim=16, rms_norm_eps=1e-6, rope_theta=1e4)
    a, _ = pm.self_attention(h, torch.arange(n), aw, cfg)
    h2, res_want = pm.add_rms_norm(a, summed, w[p + "post_attention_layernorm.weight"], 1e-6)
    gu = w[p + "mlp.gate_up.weight"]
    want = pm.gated_mlp(h2, gu[:100], gu[100:], w[p + "mlp.down.weight"])
    check(hidden, want, dtype)
    check(res, res_want, dtype)
    # the first block of a model starts the residual stream from its input
    hidden0, res0 = block.forward(ctx, x.to(DEV), None, cache)
    h0 = pm.rms_norm(x.double(), w[p + "input_layernorm.weight"], 1e-6)
    a0, _ = pm.self_attention(h0, torch.arange(n), aw, cfg)
    _, res0_want = pm.add_rms_norm(a0, x.double(), w[p + "post_attention_layernorm.weight"], 1e-6)
    check(res0, res0_want, dtype)


# ------------------------------------------------------------------ a toy mixer with a state of its own


class RunningMeanMixer(Mixer):
    """y_t = W . mean(x_0 .. x_t): the state of a request is the running sum of its inputs and the
    number of tokens seen, a fixed size whatever the context.  It reads the batch from the step's
    device arrays only and runs the same operations for every batch, so a decode step with it can be
    replayed from a captured graph; padding rows (request -1, state slot -1) change no state."""

    graph_safe = True

    def __init__(self, hidden_size: int, prefix: str = ""):
        super().__init__(prefix)
        self.hidden_size = hidden_size

    def param_specs(self):
        return {"mix.weight": ParamSpec.single("mix.weight", (self.hidden_size, self.hidden_size))}

    def cache_need(self):
        return StateNeed((self.hidden_size + 1,), torch.float32)

    def forward(self, ctx, x, cache):
        state = cache.state                                       # [slots, hidden + 1]
        seq = ctx.token_seq.long()                                # request of each token, -1 for padding
        live = (seq >= 0)
        seq = seq.clamp(min=0)
        starts = ctx.cu_seqlens_q.long()
        slot = ctx.slot_of_seq.long()
        slot_live = (slot >= 0)
        slot = slot.clamp(min=0)
        xs = x.double() * live[:, None]
        running = torch.cumsum(xs, dim=0)                         # over the whole token axis ...
        before = (running - xs).index_select(0, starts[:-1])      # ... minus what precedes each request's rows
        old = state.double().index_select(0, slot)                # [S, hidden + 1]
        sums = old[:, :-1].index_select(0, seq) + running - before.index_select(0, seq)
        rows = torch.arange(x.shape[0], device=x.device)
        counts = old[:, -1].index_select(0, seq) + (rows - starts[:-1].index_select(0, seq) + 1)
        out = (sums / counts[:, None]).to(x.dtype)
        last = (starts[1:] - 1).clamp(min=0)                      # each request's last row of this step
        new = torch.cat((sums.index_select(0, last), counts.index_select(0, last)[:, None]), dim=1)
        state.index_add_(0, slot, ((new - old) * slot_live[:, None]).float())
        return ctx.ops.linear(out, self.params["mix.weight"])


@dataclass(frozen=True)
class ToyConfig(ModelConfig):
    num_attention_heads: int = 2
    head_dim: int = 16
    intermediate_size: int = 48
    rms_norm_eps: float = 1e-5
    model_type: ClassVar[str] = "toy"

    @classmethod
    def from_dict(cls, raw):
        return cls(architecture=raw["architectures"][0], vocab_size=raw["vocab_size"], hidden_size=raw["hidden_size"],
                   num_hidden_layers=raw["num_hidden_layers"], max_position_embeddings=raw["max_position_embeddings"],
                   tie_word_embeddings=raw.get("tie_word_embeddings", False), torch_dtype="bfloat16",
                   bos_token_id=None, eos_token_id=None)

    def to_dict(self):
        return dict(architectures=[self.architecture], vocab_size=self.vocab_size, hidden_size=self.hidden_size,
                    num_hidden_layers=self.num_hidden_layers, max_position_embeddings=self.max_position_embeddings,
                    tie_word_embeddings=self.tie_word_embeddings)


def toy_spec(cfg: ToyConfig) -> ModelSpec:
    norm = PartChoice("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps})
    ffn = PartChoice("gated_mlp", {"hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size})
    attn = PartChoice("attention", {"hidden_size": cfg.hidden_size, "num_heads": cfg.num_attention_heads,
                                    "num_kv_heads": 1, "head_dim": cfg.head_dim,
                                    "position_encoding": PartChoice("rotary", {"theta": 1e4, "max_positions": cfg.max_position_embeddings})})
    toy = PartChoice("running_mean", {"hidden_size": cfg.hidden_size})
    blocks = [PartChoice("prenorm", {"mixer": toy if i % 2 == 0 else attn, "feed_forward": ffn, "norm": norm})
              for i in range(cfg.num_hidden_layers)]
    return ModelSpec(cfg.vocab_size, cfg.hidden_size, blocks, norm, max_positions=cfg.max_position_embeddings)


def plain_toy_logits(tensors, cfg: ToyConfig, ids):
    x = tensors["model.embed_tokens.weight"][torch.tensor(ids)]
    n = len(ids)
    residual = None
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        if residual is None:
            residual, h = x, pm.rms_norm(x, tensors[p + "input_layernorm.weight"], cfg.rms_norm_eps)
        else:
            h, residual = pm.add_rms_norm(x, residual, tensors[p + "input_layernorm.weight"], cfg.rms_norm_eps)
        if i % 2 == 0:
            mean = torch.cumsum(h, dim=0) / torch.arange(1, n + 1, dtype=h.dtype)[:, None]
            a = mean @ tensors[p + "self_attn.mix.weight"].T
        else:
            t = h.shape[0]
            q = (h @ tensors[p + "self_attn.q_proj.weight"].T).view(t, cfg.num_attention_heads, cfg.head_dim)
            k = (h @ tensors[p + "self_attn.k_proj.weight"].T).view(t, 1, cfg.head_dim)
            v = (h @ tensors[p + "self_attn.v_proj.weight"].T).view(t, 1, cfg.head_dim)
            cos, sin = pm.rope_angles(torch.arange(t), cfg.head_dim, 1e4)
            o = pm.causal_attention(pm.rope_neox(q, cos, sin), pm.rope_neox(k, cos, sin), v, cfg.head_dim ** -0.5)
            a = o.reshape(t, -1) @ tensors[p + "self_attn.o_proj.weight"].T
        h, residual = pm.add_rms_norm(a, residual, tensors[p + "post_attention_layernorm.weight"], cfg.rms_norm_eps)
        x = pm.gated_mlp(h, tensors[p + "mlp.gate_proj.weight"], tensors[p + "mlp.up_proj.weight"], tensors[p + "mlp.down_proj.weight"])
    h, _ = pm.add_rms_norm(x, residual, tensors["model.norm.weight"], cfg.rms_norm_eps)
    return h @ tensors["lm_head.weight"].T


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_mixer_with_state_is_registered_built_and_stepped(dtype, tmp_path):
    MIXERS.register("running_mean", RunningMeanMixer)
    register_architecture("ToyForCausalLM", ToyConfig, toy_spec)
    try:
        cfg = ToyConfig.from_dict(dict(architectures=["ToyForCausalLM"], vocab_size=97, hidden_size=40,
                                       num_hidden_layers=3, max_position_embeddings=96))
        folder = write_random_model(str(tmp_path / "toy"), cfg, seed=4, std=0.2, norm_std=0.1)
        from safetensors.torch import load_file
        tensors = {k: v.double() for k, v in load_file(folder + "/model.safetensors").items()}
        assert "model.layers.0.self_attn.mix.weight" in tensors and "model.layers.1.self_attn.q_proj.weight" in tensors
        model, loaded = load_model(folder, dtype=dtype, device=DEV)
        assert isinstance(loaded, ToyConfig) and isinstance(model.blocks[0].mixer, RunningMeanMixer)
        core = build_core(model, gpu_ops(), dtype=dtype, device=DEV, page_size=16, num_pages=12, max_num_seqs=3,
                          graph_sizes=[2])
        assert core.graphs is not None, "a model whose stateful mixer is graph safe decodes through graphs"
        assert len(core.storage.state_tensors) == 2 and core.storage.state_tensors[0].shape == (3, 41)
        g = torch.Generator().manual_seed(0)
        reqs = {r: torch.randint(0, 97, (n,), generator=g).tolist() for r, n in (("a", 50), ("b", 23), ("c", 70))}
        want = {r: plain_toy_logits(tensors, cfg, ids) for r, ids in reqs.items()}
        got = {r: {} for r in reqs}

        def step(parts):
            entries = [StepEntry(r, reqs[r][lo:hi], list(range(hi - lo))) for r, lo, hi in parts]
            logits = core.step(entries)
            at = 0
            for r, lo, hi in parts:
                for pos in range(lo, hi):
                    got[r][pos] = logits[at].cpu()
                    at += 1

        step([("a", 0, 20)])
        step([("a", 20, 21), ("b", 0, 23)])
        core.close("b")                       # b's slot goes back ...
        step([("a", 21, 40), ("c", 0, 2)])    # ... and c starts in it with a zeroed state
        assert core.manager.state_slot("c") == 1
        assert core.graphs.replays == 0
        for t in range(10):                   # both decode: a replayed graph of two rows
            step([("a", 40 + t, 41 + t), ("c", 2 + t, 3 + t)])
        core.close("a")
        step([("c", 12, 13)])                 # one request in the graph of two rows: the other row is padding
        step([("c", 13, 14)])
        assert core.graphs.replays == 12
        step([("c", 14, 70)])
        tol = 3e-5 if dtype == torch.float32 else 4e-2
        for r, ids in reqs.items():
            scale = float(want[r].abs().max())
            for pos in range(len(ids)):
                diff = float((got[r][pos].double() - want[r][pos]).abs().max())
                assert diff <= tol * scale, f"request {r} position {pos}: {diff:.3e} > {tol * scale:.3e}"
    finally:
        MIXERS.unregister("running_mean")
        unregister_architecture("ToyForCausalLM")


# ------------------------------------------------------------------ a kind of memory the framework does not know


@dataclass(frozen=True)
class PreviousTokenNeed:
    """The last input of every request: neither pages nor a ``StateNeed``."""
    width: int


@dataclass
class PreviousTokenBinding:
    last: torch.Tensor     # [slots, width] float32
    seen: torch.Tensor     # [slots] int32, tokens of the request so far


class PreviousTokenKind(CacheKind):
    def request_bytes(self, need, dtype):
        return need.width * 4 + 4

    def allocate(self, need, *, group, num_pages, page_size, num_slots, device, dtype):
        return PreviousTokenBinding(torch.full((num_slots, need.width), 7.0, device=device),   # not zero: reset must clear
                                    torch.full((num_slots,), 3, dtype=torch.int32, device=device))

    def reset(self, binding, slots):
        binding.last.index_fill_(0, slots, 0)
        binding.seen.index_fill_(0, slots, 0)


class PreviousTokenMixer(Mixer):
    """y_t = W (x_t + x_{t-1}), x_{-1} = 0; walks the requests through the step's host-side lists."""

    def __init__(self, hidden_size: int, prefix: str = ""):
        super().__init__(prefix)
        self.hidden_size = hidden_size

    def param_specs(self):
        return {"mix.weight": ParamSpec.single("mix.weight", (self.hidden_size, self.hidden_size))}

    def cache_need(self):
        return PreviousTokenNeed(self.hidden_size)

    def forward(self, ctx, x, cache):
        assert isinstance(cache, PreviousTokenBinding)
        shifted = torch.empty_like(x, dtype=torch.float32)
        for start, n, cached, slot in zip(ctx.seq_starts, ctx.seq_lens, ctx.seq_cached, ctx.state_slots):
            assert int(cache.seen[slot]) == cached
            rows = x[start:start + n].float()
            shifted[start] = cache.last[slot]
            shifted[start + 1:start + n] = rows[:-1]
            cache.last[slot] = rows[-1]
            cache.seen[slot] += n
        return ctx.ops.linear((x.float() + shifted).to(x.dtype), self.params["mix.weight"])


def previous_token_spec(cfg: ToyConfig) -> ModelSpec:
    norm = PartChoice("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps})
    ffn = PartChoice("gated_mlp", {"hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size})
    blocks = [PartChoice("prenorm", {"mixer": PartChoice("previous_token", {"hidden_size": cfg.hidden_size}),
                                     "feed_forward": ffn, "norm": norm}) for _ in range(cfg.num_hidden_layers)]
    return ModelSpec(cfg.vocab_size, cfg.hidden_size, blocks, norm, max_positions=cfg.max_position_embeddings)


def plain_previous_token_logits(tensors, cfg: ToyConfig, ids):
    x = tensors["model.embed_tokens.weight"][torch.tensor(ids)]
    residual = None
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        if residual is None:
            residual, h = x, pm.rms_norm(x, tensors[p + "input_layernorm.weight"], cfg.rms_norm_eps)
        else:
            h, residual = pm.add_rms_norm(x, residual, tensors[p + "input_layernorm.weight"], cfg.rms_norm_eps)
        a = (h + torch.cat((torch.zeros_like(h[:1]), h[:-1]))) @ tensors[p + "self_attn.mix.weight"].T
        h, residual = pm.add_rms_norm(a, residual, tensors[p + "post_attention_layernorm.weight"], cfg.rms_norm_eps)
        x = pm.gated_mlp(h, tensors[p + "mlp.gate_proj.weight"], tensors[p + "mlp.up_proj.weight"], tensors[p + "mlp.down_proj.weight"])
    h, _ = pm.add_rms_norm(x, residual, tensors["model.norm.weight"], cfg.rms_norm_eps)
    return h @ tensors["lm_head.weight"].T


def test_toy_cache_kind_is_registered_planned_and_cleared(tmp_path):
    """A mixer whose memory is of a kind defined here: the kind is registered, and planning, allocation,
    clearing for a new request and the step run without a change to the framework's files."""
    dtype = torch.float32
    MIXERS.register("previous_token", PreviousTokenMixer)
    register_cache_kind(PreviousTokenNeed, PreviousTokenKind())
    register_architecture("PreviousTokenForCausalLM", ToyConfig, previous_token_spec)
    try:
        cfg = ToyConfig.from_dict(dict(architectures=["PreviousTokenForCausalLM"], vocab_size=61, hidden_size=24,
                                       num_hidden_layers=2, max_position_embeddings=64))
        folder = write_random_model(str(tmp_path / "prev"), cfg, seed=8, std=0.3, norm_std=0.1, dtype=torch.float32)
        from safetensors.torch import load_file
        tensors = {k: v.double() for k, v in load_file(folder + "/model.safetensors").items()}
        model, _ = load_model(folder, dtype=dtype, device=DEV)
        core = build_core(model, gpu_ops(), dtype=dtype, device=DEV, page_size=16, num_pages=4, max_num_seqs=2)
        assert core.plan.groups == [] and core.plan.bytes_per_slot == 2 * (24 * 4 + 4)
        assert all(isinstance(b, PreviousTokenBinding) for b in core.storage.bindings)
        assert not core.prefix_caching and core.graphs is None
        g = torch.Generator().manual_seed(3)
        reqs = {r: torch.randint(0, 61, (n,), generator=g).tolist() for r, n in (("a", 30), ("b", 11), ("c", 9))}
        got = {r: {} for r in reqs}
        plan = [[("a", 0, 7)], [("a", 7, 8), ("b", 0, 11)], [("a", 8, 30)], [("c", 0, 1)], [("c", 1, 9)]]
        for k, parts in enumerate(plan):
            if k == 3:
                core.close("b")     # c takes b's slot, which the kind clears
            logits = core.step([StepEntry(r, reqs[r][lo:hi], list(range(hi - lo))) for r, lo, hi in parts])
            at = 0
            for r, lo, hi in parts:
                for pos in range(lo, hi):
                    got[r][pos] = logits[at].cpu()
                    at += 1
        assert core.manager.state_slot("c") == 1
        for r, ids in reqs.items():
            want = plain_previous_token_logits(tensors, cfg, ids)
            scale = float(want.abs().max())
            for pos in range(len(ids)):
                assert float((got[r][pos].double() - want[pos]).abs().max()) <= 3e-5 * scale, f"{r} position {pos}"
        with pytest.raises(KeyError):
            kind_of(object())
    finally:
        MIXERS.unregister("previous_token")
        unregister_cache_kind(PreviousTokenNeed)
        unregister_architecture("PreviousTokenForCausalLM")


# ------------------------------------------------------------------ toy parts of the other kinds: a feed-forward
# with routing, a position encoding with parameters of its own, a mixer that keeps no cache


class LearnedPositions(PositionEncoding):
    """One learned vector per position, added to the mixer's input."""

    def __init__(self, size: int, max_positions: int, prefix: str = ""):
        super().__init__(prefix)
        self.size, self.max_positions = size, max_positions

    def param_specs(self):
        return {"table": ParamSpec.single("positions.weight", (self.max_positions, self.size))}


class ShiftMixer(Mixer):
    """y_t = W (x_t + P[position of t]): no memory of other tokens, hence no cache; the position encoding is
    a child part chosen by name, with its own checkpoint tensor."""

    def __init__(self, hidden_size: int, position_encoding: PartChoice, prefix: str = ""):
        super().__init__(prefix)
        self.hidden_size = hidden_size
        self.pos = position_encoding.build(POSITION_ENCODINGS, size=hidden_size, prefix=prefix)

    def children(self):
        return [self.pos]

    def param_specs(self):
        return {"mix.weight": ParamSpec.single("mix.weight", (self.hidden_size, self.hidden_size))}

    def forward(self, ctx, x, cache):
        assert cache is None
        shifted = (x.float() + self.pos.params["table"][ctx.positions.long()].float()).to(x.dtype)
        return ctx.ops.linear(shifted, self.params["mix.weight"])


class RoutedFeedForward(FeedForward):
    """Top-1 routing over small SiLU-gated experts: router logits in float32, the chosen expert's output
    scaled by its softmax weight."""

    def __init__(self, hidden_size: int, intermediate_size: int, num_experts: int, prefix: str = ""):
        super().__init__(prefix)
        self.h, self.i, self.e = hidden_size, intermediate_size, num_experts

    def param_specs(self):
        specs = {"router.weight": ParamSpec.single("router.weight", (self.e, self.h))}
        for k in range(self.e):
            specs[f"experts.{k}.gate_up.weight"] = ParamSpec.stacked(
                [(f"experts.{k}.gate_proj.weight", self.i), (f"experts.{k}.up_proj.weight", self.i)], (self.h,))
            specs[f"experts.{k}.down.weight"] = ParamSpec.single(f"experts.{k}.down_proj.weight", (self.h, self.i))
        return specs

    def forward(self, ctx, x):
        ops = ctx.ops
        logits = ops.linear(x, self.params["router.weight"], None, out_dtype=torch.float32)
        weight, choice = torch.softmax(logits, dim=-1).max(dim=-1)
        out = torch.zeros_like(x)
        for k in range(self.e):
            rows = (choice == k).nonzero().squeeze(1)
            if rows.numel() == 0:
                continue
            act = ops.linear_silu(x[rows].contiguous(), self.params[f"experts.{k}.gate_up.weight"])
            y = ops.materialize(ops.linear(act, self.params[f"experts.{k}.down.weight"]))
            out[rows] = (y.float() * weight[rows, None]).to(x.dtype)
        return out


def routed_spec(cfg: ToyConfig) -> ModelSpec:
    norm = PartChoice("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps})
    dense = PartChoice("gated_mlp", {"hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size})
    routed = PartChoice("routed_toy", {"hidden_size": cfg.hidden_size, "intermediate_size": 24, "num_experts": 3})
    attn = PartChoice("attention", {"hidden_size": cfg.hidden_size, "num_heads": cfg.num_attention_heads,
                                    "num_kv_heads": 2, "head_dim": cfg.head_dim,
                                    "position_encoding": PartChoice("rotary", {"theta": 1e4, "max_positions": cfg.max_position_embeddings})})
    shift = PartChoice("shift_toy", {"hidden_size": cfg.hidden_size, "position_encoding": PartChoice(
        "learned_toy", {"max_positions": cfg.max_position_embeddings})})
    blocks = [PartChoice("prenorm", {"mixer": shift if i % 2 == 0 else attn, "feed_forward": routed if i % 2 == 0 else dense,
                                     "norm": norm}) for i in range(cfg.num_hidden_layers)]
    return ModelSpec(cfg.vocab_size, cfg.hidden_size, blocks, norm, max_positions=cfg.max_position_embeddings)


def plain_routed_logits(tensors, cfg: ToyConfig, ids, round_to=None):
    x = tensors["model.embed_tokens.weight"][torch.tensor(ids)]
    n = len(ids)
    residual = None
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        if residual is None:
            residual, h = x, pm.rms_norm(x, tensors[p + "input_layernorm.weight"], cfg.rms_norm_eps)
        else:
            h, residual = pm.add_rms_norm(x, residual, tensors[p + "input_layernorm.weight"], cfg.rms_norm_eps)
        if i % 2 == 0:
            a = (h + tensors[p + "self_attn.positions.weight"][:n]) @ tensors[p + "self_attn.mix.weight"].T
        else:
            q = (h @ tensors[p + "self_attn.q_proj.weight"].T).view(n, cfg.num_attention_heads, cfg.head_dim)
            k = (h @ tensors[p + "self_attn.k_proj.weight"].T).view(n, 2, cfg.head_dim)
            v = (h @ tensors[p + "self_attn.v_proj.weight"].T).view(n, 2, cfg.head_dim)
            cos, sin = pm.rope_angles(torch.arange(n), cfg.head_dim, 1e4)
            o = pm.causal_attention(pm.rope_neox(q, cos, sin), pm.rope_neox(k, cos, sin), v, cfg.head_dim ** -0.5)
            a = o.reshape(n, -1) @ tensors[p + "self_attn.o_proj.weight"].T
        h, residual = pm.add_rms_norm(a, residual, tensors[p + "post_attention_layernorm.weight"], cfg.rms_norm_eps)
        if i % 2 == 0:
            probs = torch.softmax(h @ tensors[p + "mlp.router.weight"].T, dim=-1)
            weight, choice = probs.max(dim=-1)
            x = torch.zeros_like(h)
            for t in range(n):
                e = int(choice[t])
                pre = f"{p}mlp.experts.{e}."
                x[t] = weight[t] * pm.gated_mlp(h[t:t + 1], tensors[pre + "gate_proj.weight"], tensors[pre + "up_proj.weight"],
                                                tensors[pre + "down_proj.weight"])[0]
        else:
            x = pm.gated_mlp(h, tensors[p + "mlp.gate_proj.weight"], tensors[p + "mlp.up_proj.weight"],
                             tensors[p + "mlp.down_proj.weight"])
    h, _ = pm.add_rms_norm(x, residual, tensors["model.norm.weight"], cfg.rms_norm_eps)
    return h @ tensors["lm_head.weight"].T


def test_toy_routed_feed_forward_and_learned_positions(tmp_path):
    """float32 only: with 8-bit mantissas a router's top-1 choice can flip on near ties, which is a
    property of routing and not of the engine."""
    dtype = torch.float32
    MIXERS.register("shift_toy", ShiftMixer)
    FEED_FORWARDS.register("routed_toy", RoutedFeedForward)
    POSITION_ENCODINGS.register("learned_toy", LearnedPositions)
    register_architecture("RoutedToyForCausalLM", ToyConfig, routed_spec)
    try:
        cfg = ToyConfig.from_dict(dict(architectures=["RoutedToyForCausalLM"], vocab_size=83, hidden_size=32,
                                       num_hidden_layers=4, max_position_embeddings=80))
        folder = write_random_model(str(tmp_path / "routed"), cfg, seed=6, std=0.25, norm_std=0.1, dtype=torch.float32)
        from safetensors.torch import load_file
        tensors = {k: v.double() for k, v in load_file(folder + "/model.safetensors").items()}
        for name in ("model.layers.0.self_attn.positions.weight", "model.layers.2.mlp.router.weight",
                     "model.layers.0.mlp.experts.2.up_proj.weight", "model.layers.1.mlp.gate_proj.weight"):
            assert name in tensors
        model, _ = load_model(folder, dtype=dtype, device=DEV)
        core = build_core(model, gpu_ops(), dtype=dtype, device=DEV, page_size=16, num_pages=10, max_num_seqs=2)
        assert core.storage.bindings[0] is None and core.storage.bindings[1] is not None   # only attention keeps pages
        g = torch.Generator().manual_seed(1)
        reqs = {r: torch.randint(0, 83, (n,), generator=g).tolist() for r, n in (("a", 60), ("b", 33))}
        got = {r: {} for r in reqs}
        plan = [[("a", 0, 17)], [("a", 17, 18), ("b", 0, 30)], [("a", 18, 60), ("b", 30, 31)], [("b", 31, 33)]]
        for parts in plan:
            logits = core.step([StepEntry(r, reqs[r][lo:hi], list(range(hi - lo))) for r, lo, hi in parts])
            at = 0
            for r, lo, hi in parts:
                for pos in range(lo, hi):
                    got[r][pos] = logits[at].cpu()
                    at += 1
        experts_used = set()
        for r, ids in reqs.items():
            want = plain_routed_logits(tensors, cfg, ids)
            scale = float(want.abs().max())
            for pos in range(len(ids)):
                diff = float((got[r][pos].double() - want[pos]).abs().max())
                assert diff <= 5e-5 * scale, f"request {r} position {pos}: {diff:.3e}"
        # the routing did route: more than one expert was chosen in the first layer
        h = pm.rms_norm(tensors["model.embed_tokens.weight"][torch.tensor(reqs["a"])], tensors["model.layers.0.input_layernorm.weight"], 1e-5)
        a = (h + tensors["model.layers.0.self_attn.positions.weight"][:60]) @ tensors["model.layers.0.self_attn.mix.weight"].T
        h2, _ = pm.add_rms_norm(a, tensors["model.embed_tokens.weight"][torch.tensor(reqs["a"])],
                                tensors["model.layers.0.post_attention_layernorm.weight"], 1e-5)
        experts_used = set((h2 @ tensors["model.layers.0.mlp.router.weight"].T).argmax(-1).tolist())
        assert len(experts_used) >= 2
    finally:
        MIXERS.unregister("shift_toy")
        FEED_FORWARDS.unregister("routed_toy")
        POSITION_ENCODINGS.unregister("learned_toy")
        unregister_architecture("RoutedToyForCausalLM")


# ------------------------------------------------------------------ an embedding and a head with kernels of their own


TOY_KERNELS = [__file__.rsplit("/", 1)[0] + "/toy_kernels.hip"]


def _toy_lib(ops):
    """The toy parts' own HIP kernels: compiled with the framework's flags on first use, bound here."""
    import ctypes
    lib = ops.load_extension(TOY_KERNELS, "libtoy_kernels.so")
    lib.toy_scale.restype = lib.toy_softcap.restype = ctypes.c_int
    return lib


class ScaledEmbedding(TokenEmbedding):
    """The table's rows times a constant (as architectures that scale their embedding by sqrt(hidden) do)."""

    def __init__(self, vocab_size, hidden_size, multiplier: float, prefix=""):
        super().__init__(vocab_size, hidden_size, prefix)
        self.multiplier = float(multiplier)

    def forward(self, ctx, ids):
        import ctypes
        x = super().forward(ctx, ids)
        ctx.ops.check("embedded rows", x, (torch.float32, torch.bfloat16), (ids.numel(), self.hidden_size))
        status = _toy_lib(ctx.ops).toy_scale(ctx.ops.pointer(x), ctypes.c_long(x.numel()), ctypes.c_float(self.multiplier),
                                             int(x.dtype == torch.bfloat16), ctx.ops.stream())
        assert status == 0
        return x


class CappedHead(LMHead):
    """``cap * tanh(logits / cap)``: a soft cap on the logits."""

    def __init__(self, vocab_size, hidden_size, cap: float, tied_to=None, prefix=""):
        super().__init__(vocab_size, hidden_size, tied_to, prefix)
        self.cap = float(cap)

    def forward(self, ctx, x):
        import ctypes
        logits = super().forward(ctx, x)
        ctx.ops.check("logits", logits, torch.float32, (x.shape[0], self.vocab_size))
        status = _toy_lib(ctx.ops).toy_softcap(ctx.ops.pointer(logits), ctypes.c_long(logits.numel()),
                                               ctypes.c_float(self.cap), ctx.ops.stream())
        assert status == 0
        return logits


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_and_head_with_kernels_of_their_own(dtype, tmp_path):
    """The embedding and the head come from registries like every other part, and a part may bring HIP code of its
    own: both toys are defined here, their kernels lie beside this file, and the model that uses them is built,
    loaded and stepped (decode steps through replayed graphs) without a change to the framework's files."""
    import dataclasses

    from atom_amd.config.model_config import Qwen3Config
    from atom_amd.models.qwen3 import qwen3_spec
    from atom_amd.parts import EMBEDDINGS, HEADS
    from tiny import TINY_B

    multiplier, cap = 96 ** 0.5, 0.7

    def capped_spec(cfg):
        return dataclasses.replace(qwen3_spec(cfg), embedding=PartChoice("scaled_embedding", {"multiplier": multiplier}),
                                   head=PartChoice("capped_head", {"cap": cap}))

    EMBEDDINGS.register("scaled_embedding", ScaledEmbedding)
    HEADS.register("capped_head", CappedHead)
    register_architecture("ToyCappedForCausalLM", Qwen3Config, capped_spec)
    try:
        raw = dict(TINY_B, architectures=["ToyCappedForCausalLM"])
        cfg = Qwen3Config.from_dict(raw)
        folder = write_random_model(str(tmp_path / "capped"), cfg, seed=6, std=0.05, norm_std=0.2)
        model, _ = load_model(folder, dtype=dtype, device=DEV)
        assert isinstance(model.embedding, ScaledEmbedding) and isinstance(model.head, CappedHead)
        core = build_core(model, gpu_ops(), dtype=dtype, device=DEV, page_size=8, num_pages=24, max_num_seqs=2,
                          graph_sizes=[1, 2])
        ids = torch.randint(0, cfg.vocab_size, (60,), generator=torch.Generator().manual_seed(3)).tolist()
        # the plain implementation with the table scaled beforehand and the cap applied afterwards
        plain_cfg, tensors = pm.load_folder(folder)
        tensors = dict(tensors)
        tensors["model.embed_tokens.weight"] = tensors["model.embed_tokens.weight"] * multiplier
        raw_logits = pm.qwen3_logits(plain_cfg, tensors, ids)
        want = cap * torch.tanh(raw_logits / cap)
        assert float(raw_logits.abs().max()) > 1.5 * cap, "the cap must bite for the test to mean something"
        got = [core.step([StepEntry("r", ids[:40], list(range(40)))]).cpu()]
        for t in range(40, 60):
            got.append(core.step([StepEntry("r", [ids[t]], [0])]).cpu())
        assert core.graphs is not None and core.graphs.replays == 20
        got = torch.cat(got).double()
        tol = 1e-4 if dtype == torch.float32 else 4e-2
        assert float((got - want).abs().max()) <= tol * cap
    finally:
        EMBEDDINGS.unregister("scaled_embedding")
        HEADS.unregister("capped_head")
        unregister_architecture("ToyCappedForCausalLM")
