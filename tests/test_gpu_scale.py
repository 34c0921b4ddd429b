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
    """48 requests of different lengths decode together (the library's products, attention parts merged
    inside a block); each row equals the request decoded alone (the skinny kernel, the merge kernel)."""
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
