"""The serving sizes: two layers of the Qwen3-8B shape (hidden 4096, 32/8 heads of 128, 12288 wide,
151,936 tokens) with random weights, thousands of cached tokens, dozens of live requests.  No plain
implementation runs at this size in reasonable time, so the engine is compared with itself: the same
requests whole, in portions, token by token through the decode graphs, and mixed, in bfloat16 within the
tolerance of the replay tests; and one request in true 32-bit against bfloat16.  What this catches is
what tiny models cannot show: offsets beyond 32 bits, grids and workspaces at real sizes, kernel paths
that only large products take (the library's products, the skinny kernel's wide mode, tiled prefill)."""

import pytest
import torch

from helpers import gpu_ops
from replay import TOL
from atom_amd.config import model_config_from_dict
from atom_amd.config.registry import build_model
from atom_amd.engine.core import StepEntry, build_core
from atom_amd.weights.loader import load_weights
from atom_amd.weights.random_init import RandomSource

pytestmark = pytest.mark.gpu

SHAPE = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=2, hidden_size=4096,
             num_attention_heads=32, num_key_value_heads=8, head_dim=128, intermediate_size=12288, vocab_size=151936,
             rope_theta=1000000.0, rms_norm_eps=1e-6, max_position_embeddings=40960, tie_word_embeddings=False,
             attention_bias=False, use_sliding_window=False, hidden_act="silu", torch_dtype="bfloat16")
LAST = 24   # positions at the end of each request whose logits are compared


def _core(dtype, **kw):
    cfg = model_config_from_dict(dict(SHAPE))
    model = build_model(cfg)
    load_weights(model, RandomSource(model, 5, device="cuda:0"), "cuda:0", dtype, None)
    kw.setdefault("num_pages", 2048)
    kw.setdefault("max_num_seqs", 64)
    return build_core(model, gpu_ops(), dtype=dtype, device="cuda:0", page_size=16, max_model_len=8192, **kw)


def _ids(n, seed):
    return torch.randint(0, SHAPE["vocab_size"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def _close(got, want, dtype, what):
    scale = float(want.abs().max())
    diff = (got.double() - want.double()).abs()
    tol = TOL[dtype]
    assert torch.isfinite(got).all(), what
    assert float(diff.max()) <= tol["max"] * scale and float(diff.mean()) <= tol["mean"] * scale, \
        f"{what}: max diff {float(diff.max()):.3e}, mean {float(diff.mean()):.3e}, scale {scale:.3f}"


def test_cuts_agree_at_serving_sizes():
    core = _core(torch.bfloat16, graph_sizes=[1, 4, 8])
    requests = {"a": _ids(2500, 1), "b": _ids(700, 2), "c": _ids(1300, 3)}
    whole = {}
    for rid, ids in requests.items():
        whole[rid] = core.step([StepEntry(rid, ids, list(range(len(ids) - LAST, len(ids))))]).cpu()
        core.close(rid)

    # most of each prompt in one step, then the three requests decode together (a graph of eight rows)
    for rid, ids in requests.items():
        core.step([StepEntry(rid, ids[:-LAST], [])])
    rows = {rid: [] for rid in requests}
    for t in range(LAST):
        out = core.step([StepEntry(rid, [ids[len(ids) - LAST + t]], [0]) for rid, ids in requests.items()])
        for k, rid in enumerate(requests):
            rows[rid].append(out[k].cpu())
    assert core.graphs.replays == LAST
    for rid in requests:
        _close(torch.stack(rows[rid]), whole[rid], "bfloat16", f"decoded tail of {rid}")
        core.close(rid)

    # portions of 512 and 96 tokens; the last portion of one request beside single tokens of another
    for rid, ids in requests.items():
        at, size, got = 0, 512, []
        while at < len(ids):
            n = min(size, len(ids) - at)
            want = [i - at for i in range(max(at, len(ids) - LAST), at + n)]
            out = core.step([StepEntry(rid, ids[at:at + n], want)])
            if want:
                got.append(out.cpu())
            at += n
            size = 96 if size == 512 else 512
        _close(torch.cat(got), whole[rid], "bfloat16", f"portions of {rid}")
        core.close(rid)
    a, b = requests["a"], requests["b"]
    core.step([StepEntry("b", b[:-LAST], [])])
    core.step([StepEntry("a", a[:2000], [])])
    got_a, got_b = [], []
    at = 2000
    for t in range(LAST):
        entries = [StepEntry("b", [b[len(b) - LAST + t]], [0])]
        if at < len(a):
            n = min(64, len(a) - at)
            entries.append(StepEntry("a", a[at:at + n], [i - at for i in range(max(at, len(a) - LAST), at + n)]))
        out = core.step(entries).cpu()
        got_b.append(out[0])
        if len(entries) == 2:
            if out.shape[0] > 1:
                got_a.append(out[1:])
            at += n
    _close(torch.stack(got_b), whole["b"], "bfloat16", "b decoded beside portions of a")
    _close(torch.cat(got_a), whole["a"], "bfloat16", "portions of a beside b's tokens")
    core.manager.check()


def test_many_live_requests_decode_like_each_alone():
    """48 requests of different lengths decode together (the product kernel for 17 to 64 rows, attention parts
    merged inside a block); each row equals the request decoded alone (the kernel for up to 16 rows, the merge kernel)."""
    core = _core(torch.bfloat16, graph_sizes=[1, 64], num_pages=4096)
    lens = [17 + 53 * k for k in range(48)]
    prompts = {f"r{k}": _ids(n, 100 + k) for k, n in enumerate(lens)}
    nxt = {rid: _ids(3, 900 + k) for k, rid in enumerate(prompts)}
    for rid, ids in prompts.items():
        core.step([StepEntry(rid, ids, [])])
    together = [core.step([StepEntry(rid, [nxt[rid][t]], [0]) for rid in prompts]).cpu() for t in range(3)]
    for rid in prompts:
        core.close(rid)
    for k, rid in list(enumerate(prompts))[::5]:
        core.step([StepEntry(rid, prompts[rid], [])])
        for t in range(3):
            alone = core.step([StepEntry(rid, [nxt[rid][t]], [0])]).cpu()
            _close(together[t][k:k + 1], alone, "bfloat16", f"{rid} ({lens[k]} tokens), token {t}")
        core.close(rid)


def test_32_bit_and_bfloat16_agree_at_serving_sizes():
    ids = _ids(600, 7)
    want = list(range(len(ids) - LAST, len(ids)))
    wide = _core(torch.float32, num_pages=128, max_num_seqs=2).step([StepEntry("x", ids, want)]).cpu()
    torch.cuda.empty_cache()
    half = _core(torch.bfloat16, num_pages=128, max_num_seqs=2).step([StepEntry("x", ids, want)]).cpu()
    _close(half, wide, "bfloat16", "bfloat16 against 32-bit")
    assert (half.argmax(-1) == wide.argmax(-1)).float().mean() >= 0.7


def test_pages_far_into_a_large_cache():
    """A cache of 140,000 pages (4.6 GB each for keys and values): pages whose offsets no 32-bit number
    holds are written and read like the first ones (rotation + cache write, decode and prefill attention)."""
    from atom_amd.kernels.hip import AttentionMeta

    ops, dev = gpu_ops(), "cuda:0"
    hq, hkv, d, page, base = 32, 8, 128, 16, 139_000
    gen = torch.Generator().manual_seed(4)
    lens = [1000, 37]            # two requests decode; a third brings a prompt portion of 300 tokens after 212 cached
    pages_of = [63, 3, 32]
    first = [0, 63, 66]

    def run(offset, num_pages):
        kc = torch.zeros(num_pages, hkv, page, d, dtype=torch.bfloat16, device=dev)
        vc = torch.zeros(num_pages, hkv, d, page, dtype=torch.bfloat16, device=dev)
        g = torch.Generator().manual_seed(4)
        total = sum(pages_of)
        kc[offset:offset + total] = (torch.randn(total, hkv, page, d, generator=g) * 0.5).to(torch.bfloat16).to(dev)
        vc[offset:offset + total] = (torch.randn(total, hkv, d, page, generator=g) * 0.5).to(torch.bfloat16).to(dev)
        tokens = 300 + 2
        qkv = (torch.randn(tokens, (hq + 2 * hkv) * d, generator=g) * 0.5).to(torch.bfloat16).to(dev)
        width = max(pages_of)
        bt = torch.zeros(3, width, dtype=torch.int32)
        for r in range(3):
            bt[r, :pages_of[r]] = torch.arange(pages_of[r]) + offset + first[r]
        # token order: the prompt portion first (request 2), then the two decode rows (requests 0 and 1)
        order = [2, 0, 1]
        bt = bt[order].contiguous().to(dev)
        ctx = [512, lens[0], lens[1]]
        positions = torch.tensor(list(range(212, 512)) + [lens[0] - 1, lens[1] - 1], dtype=torch.int32)
        token_seq = torch.tensor([0] * 300 + [1, 2], dtype=torch.int32)
        slots = torch.tensor([int(bt[s, p // page]) * page + p % page for s, p in zip(token_seq.tolist(), positions.tolist())],
                             dtype=torch.int32).to(dev)
        half = d // 2
        inv = 1.0 / (1e6 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
        ang = torch.arange(1024, dtype=torch.float32)[:, None] * inv[None, :]
        cos, sin = ang.cos().to(dev), ang.sin().to(dev)
        w = torch.ones(d, device=dev)
        q = torch.empty(tokens, hq, d, dtype=torch.bfloat16, device=dev)
        ops.qk_norm_rope_kv_write(qkv, q, kc, vc, w, w, cos, sin, positions.to(dev), slots, hq, hkv, d, d, page, 1e-6)
        tiles = {rows: torch.tensor([(0, r) for r in range(0, 300, rows)], dtype=torch.int32, device=dev)
                 for rows in (32, 64, 128)}
        meta = AttentionMeta(token_seq=token_seq.to(dev), positions=positions.to(dev), block_tables=bt,
                             cu_seqlens_q=torch.tensor([0, 300, 301, 302], dtype=torch.int32, device=dev),
                             context_lens=torch.tensor(ctx, dtype=torch.int32, device=dev), num_seqs=3, num_tokens=tokens,
                             max_q_len=300, max_context_len=1000, page_size=page, num_prefill=1,
                             prefill_tiles=tiles[32], rows_per_tile=32, tiles_by_rows=tiles)
        out = torch.empty_like(q)
        ops.paged_attention(q, kc, vc, out, meta, d ** -0.5)
        torch.cuda.synchronize()
        written = (kc[offset + first[2] + 13:offset + first[2] + 32].clone(), vc[offset + first[2] + 13:offset + first[2] + 32].clone())
        return out.cpu(), written[0].cpu(), written[1].cpu()

    low = run(0, 128)
    torch.cuda.empty_cache()
    high = run(base, base + 128)
    assert (base + 100) * hkv * page * d > 2 ** 31
    for a, b in zip(low, high):
        assert torch.isfinite(a.float()).all() and torch.equal(a, b)
    assert float(low[0].float().abs().max()) > 0 and float(low[1].float().abs().max()) > 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_serving_layer_sizes_against_the_plain_implementation(dtype, tmp_path_factory):
    """Two layers of the full layer shape (hidden 4096, 32/8 heads of 128, 12288 wide; a small vocabulary so
    that the plain implementation's head stays cheap) written as a model folder, run by the engine (most of a
    500-token prompt in one step, the last tokens one by one) and by the plain implementation on the CPU in
    float64, which reads the same folder."""
    import plain_model
    from atom_amd.engine.core import TORCH_DTYPES, load_model
    from atom_amd.weights import write_random_model

    folder = getattr(test_serving_layer_sizes_against_the_plain_implementation, "folder", None)
    if folder is None:
        cfg = model_config_from_dict({**SHAPE, "vocab_size": 8209})
        folder = write_random_model(str(tmp_path_factory.mktemp("layers8b") / "m"), cfg, 9, 0.02, 0.1, torch.bfloat16)
        test_serving_layer_sizes_against_the_plain_implementation.folder = folder
        plain_cfg, tensors = plain_model.load_folder(folder)
        ids = torch.randint(0, 8209, (500,), generator=torch.Generator().manual_seed(3)).tolist()
        test_serving_layer_sizes_against_the_plain_implementation.ids = ids
        test_serving_layer_sizes_against_the_plain_implementation.want = plain_model.qwen3_logits(plain_cfg, tensors, ids)[-LAST:]
        del tensors
    ids = test_serving_layer_sizes_against_the_plain_implementation.ids
    want = test_serving_layer_sizes_against_the_plain_implementation.want
    model, _ = load_model(folder, dtype=TORCH_DTYPES[dtype], device="cuda:0")
    core = build_core(model, gpu_ops(), dtype=TORCH_DTYPES[dtype], device="cuda:0", page_size=16, num_pages=64,
                      max_num_seqs=2, max_model_len=1024, graph_sizes=[1])
    head = len(ids) - LAST // 2
    first = core.step([StepEntry("x", ids[:head], list(range(len(ids) - LAST, head)))]).cpu()
    rows = [first] + [core.step([StepEntry("x", [tok], [0])]).cpu() for tok in ids[head:]]
    assert core.graphs.replays == LAST // 2
    _close(torch.cat(rows), want, dtype, f"{dtype} engine against the plain implementation")
