"""Each HIP kernel alone against its plain reference, at sizes other than the engine's:
widths and vocabularies that are no power of two, head sizes in steps of 16, odd numbers
of heads and groups, several page sizes."""

import math

import pytest
import torch

from helpers import gpu_ops
from plain_kernels import PlainKernels, exponential_noise_row
from atom_amd.kernels.hip import AttentionMeta, KernelError

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PLAIN = PlainKernels()
DTYPES = [torch.float32, torch.bfloat16]


def rnd(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def close(got, want, dtype, scale=None):
    got, want = got.detach().cpu().double(), want.detach().cpu().double()
    scale = scale or max(1e-6, float(want.abs().max()))
    tol = 2e-6 if dtype == torch.float32 else 1.2e-2   # a few ulp of the output's type
    worst = float((got - want).abs().max())
    assert worst <= tol * scale, f"max diff {worst:.3e} > {tol * scale:.3e}"


@pytest.mark.parametrize("tdtype", DTYPES)
@pytest.mark.parametrize("odtype", DTYPES)
def test_embedding(tdtype, odtype):
    table = rnd((311, 136), tdtype, 0)
    ids = torch.tensor([0, 310, 5, 5, 17, 200], dtype=torch.int32)
    out = torch.empty((6, 136), dtype=odtype, device=DEV)
    gpu_ops().embedding(table.to(DEV), ids.to(DEV), out)
    want = torch.empty((6, 136), dtype=odtype)
    PLAIN.embedding(table, ids, want)
    assert torch.equal(out.cpu(), want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [16, 136, 4096, 5000, 5001, 20000])
@pytest.mark.parametrize("mode", ["plain", "init", "add"])
def test_rmsnorm(dtype, width, mode):
    rows = 7
    x = rnd((rows, width), dtype, 1, 3.0)
    w = 1 + rnd((width,), torch.float32, 2, 0.2)
    res = rnd((rows, width), torch.float32, 3, 2.0)
    out = torch.empty_like(x, device=DEV)
    res_gpu = res.to(DEV)
    gpu_ops().rmsnorm(x.to(DEV), w.to(DEV), 1e-5, out, residual=res_gpu if mode != "plain" else None, mode=mode)
    want = torch.empty_like(x)
    res_want = res.clone()
    PLAIN.rmsnorm(x, w, 1e-5, want, residual=res_want if mode != "plain" else None, mode=mode)
    close(out, want, dtype)
    if mode != "plain":
        close(res_gpu, res_want, torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_rows(dtype):
    x = rnd((9, 200), dtype, 4)
    res = rnd((9, 200), torch.float32, 5)
    w = 1 + rnd((200,), torch.float32, 6, 0.3)
    rows = torch.tensor([8, 0, 3], dtype=torch.int32)
    out = torch.empty((3, 200), dtype=dtype, device=DEV)
    res_gpu = res.to(DEV)
    gpu_ops().rmsnorm(x.to(DEV), w.to(DEV), 1e-6, out, residual=res_gpu, mode="add", rows=rows.to(DEV))
    want = torch.empty((3, 200), dtype=dtype)
    PLAIN.rmsnorm(x, w, 1e-6, want, residual=res.clone(), mode="add", rows=rows)
    close(out, want, dtype)
    assert torch.equal(res_gpu.cpu(), res), "the residual stream must stay as it was"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("inter", [333, 200, 1032])
def test_silu_mul(dtype, inter):
    x = rnd((5, 2 * inter), dtype, 7, 2.0)
    out = torch.empty((5, inter), dtype=dtype, device=DEV)
    gpu_ops().silu_mul(x.to(DEV), out)
    want = torch.empty((5, inter), dtype=dtype)
    PLAIN.silu_mul(x, want)
    close(out, want, dtype)
    swapped = torch.cat((x[:, inter:], x[:, :inter]), dim=1)
    other = torch.empty((5, inter), dtype=dtype)
    PLAIN.silu_mul(swapped, other)
    assert (other.float() - want.float()).abs().max() > 0.1, "gate and up must not be interchangeable"


@pytest.mark.parametrize("xd,wd", [(torch.float32, torch.float32), (torch.bfloat16, torch.float32),
                                   (torch.float32, torch.bfloat16), (torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("m,n,k", [(1, 311, 96), (7, 64, 130), (70, 200, 65), (3, 1, 17)])
def test_gemm_f32_kernel(xd, wd, m, n, k):
    ops = gpu_ops()
    x, w, b = rnd((m, k), xd, 8), rnd((n, k), wd, 9), rnd((n,), torch.float32, 10)
    ops.allow_library_gemm = False
    try:
        y = ops.linear(x.to(DEV), w.to(DEV), b.to(DEV), out_dtype=torch.float32)
    finally:
        ops.allow_library_gemm = True
    want = PLAIN.linear(x, w, b, out_dtype=torch.float32)
    close(y, want, torch.float32, scale=float(want.abs().max()) * 2)


def test_gemm_f32_rows_do_not_depend_on_batch():
    ops = gpu_ops()
    x, w = rnd((70, 300), torch.float32, 11).to(DEV), rnd((129, 300), torch.float32, 12).to(DEV)
    whole = ops.linear(x, w)
    for lo, hi in ((0, 1), (5, 6), (63, 70), (10, 40)):
        assert torch.equal(ops.linear(x[lo:hi].contiguous(), w), whole[lo:hi])


def test_linear_bf16_library_path():
    ops = gpu_ops()
    x, w, b = rnd((33, 136), torch.bfloat16, 13), rnd((517, 136), torch.bfloat16, 14), rnd((517,), torch.float32, 15)
    y = ops.linear(x.to(DEV), w.to(DEV), b.to(DEV))
    close(y, PLAIN.linear(x, w, b), torch.bfloat16)
    y32 = ops.linear(x.to(DEV), w.to(DEV), None, out_dtype=torch.float32)
    assert y32.dtype == torch.float32


def test_float32_logits_keep_their_precision_with_many_rows():
    """A head's float32 output is the float32 sum whatever the number of rows (few rows: the engine's own
    kernel, many: the library's), so a request's logits do not lose bits when it decodes beside many others;
    and a bias is added before the product is rounded to bfloat16."""
    ops = gpu_ops()
    x, w = rnd((150, 264), torch.bfloat16, 21), rnd((5001, 264), torch.bfloat16, 22, 0.05)
    want = x.double() @ w.double().T
    scale = float(want.abs().max())
    many = ops.linear(x.to(DEV), w.to(DEV), None, out_dtype=torch.float32)
    assert not ops._skinny(x.to(DEV), w.to(DEV))
    assert float((many.cpu().double() - want).abs().max()) <= 2e-6 * scale
    for row in (0, 77, 149):
        alone = ops.linear(x[row:row + 1].to(DEV).contiguous(), w.to(DEV), None, out_dtype=torch.float32)
        assert float((alone[0] - many[row]).abs().max()) <= 2e-6 * scale
    b = rnd((5001,), torch.float32, 23, 2.0)
    y = ops.linear(x.to(DEV), w.to(DEV), b.to(DEV))
    exact = (want + b.double()).float().to(torch.bfloat16)      # one rounding of the exact sum
    off = (y.cpu().float() - exact.float()).abs()
    assert float((off / exact.float().abs().clamp(min=1e-3)).max()) <= 2.0 ** -7, "at most one bfloat16 step off"
    assert float((off > 0).float().mean()) < 0.02, "only sums that lie at a rounding boundary may differ"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hq,hkv,d,rot,page", [(4, 2, 16, 16, 16), (6, 3, 32, 32, 8), (5, 5, 48, 24, 4),
                                              (8, 1, 128, 128, 32), (3, 1, 80, 0, 16), (5, 2, 64, 64, 16),
                                              (2, 1, 256, 256, 8), (3, 3, 96, 96, 16), (4, 2, 64, 64, 6)])
@pytest.mark.parametrize("norm", [True, False])
@pytest.mark.parametrize("tokens", [11, 45])   # 32 tokens and more take the vector kernel where it applies
def test_qk_norm_rope_kv_write(dtype, hq, hkv, d, rot, page, norm, tokens):
    pages, max_pos = -(-64 // page), 50
    qkv = rnd((tokens, (hq + 2 * hkv) * d), dtype, 16, 2.0)
    qw = 1 + rnd((d,), torch.float32, 17, 0.2) if norm else None
    kw = 1 + rnd((d,), torch.float32, 18, 0.2) if norm else None
    ang = torch.outer(torch.arange(max_pos, dtype=torch.float32), 1.0 / (1e4 ** (torch.arange(0, max(rot, 2), 2) / max(rot, 2))))
    cos, sin = ang.cos().contiguous(), ang.sin().contiguous()
    positions = torch.tensor(([3, 4, 5, 0, 1, 49, 20, 21, 22, 23, 7] * 5)[:tokens], dtype=torch.int32)
    perm = torch.randperm(pages * page, generator=torch.Generator().manual_seed(19))[:tokens].to(torch.int32)
    slots = perm.clone()
    slots[4] = -1   # a padding row writes nothing
    kc = rnd((pages, hkv, page, d), dtype, 20)
    vc = rnd((pages, hkv, d, page), dtype, 21)
    kc_gpu, vc_gpu = kc.to(DEV), vc.to(DEV)
    q_gpu = torch.empty((tokens, hq, d), dtype=dtype, device=DEV)
    dev = lambda t: t.to(DEV) if t is not None else None   # noqa: E731
    gpu_ops().qk_norm_rope_kv_write(qkv.to(DEV), q_gpu, kc_gpu, vc_gpu, dev(qw), dev(kw), cos.to(DEV), sin.to(DEV),
                                    positions.to(DEV), slots.to(DEV), hq, hkv, d, rot, page, 1e-5)
    q_want = torch.empty((tokens, hq, d), dtype=dtype)
    PLAIN.qk_norm_rope_kv_write(qkv, q_want, kc, vc, qw, kw, cos, sin, positions, slots, hq, hkv, d, rot, page, 1e-5)
    close(q_gpu, q_want, dtype)
    close(kc_gpu, kc, dtype)
    close(vc_gpu, vc, dtype)
    # reading another run's cache: nothing is written
    before_k, before_v = kc_gpu.clone(), vc_gpu.clone()
    gpu_ops().qk_norm_rope_kv_write(qkv.to(DEV), q_gpu, kc_gpu, vc_gpu, dev(qw), dev(kw), cos.to(DEV), sin.to(DEV),
                                    positions.to(DEV), slots.to(DEV), hq, hkv, d, rot, page, 1e-5, write_kv=False)
    assert torch.equal(before_k, kc_gpu) and torch.equal(before_v, vc_gpu)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page", [8, 16, 32])
def test_kv_write_of_token_runs(dtype, page):
    """Runs of 8 tokens whose slots are 8 consecutive aligned places are written together; runs that are
    shifted, broken by a padding row, cross a page or are cut short by the end take the single-token way."""
    hq, hkv, d = 4, 2, 64
    runs = [list(range(32, 40)), list(range(65, 73)), [96, 97, 98, -1, 100, 101, 102, 103],
            list(range(156, 164)),   # crosses the page edge at 160
            list(range(200, 208)), [16, 17, 18]]
    slots = torch.tensor([s for run in runs for s in run], dtype=torch.int32)
    tokens = slots.numel()
    pages = 256 // page + 2
    qkv = rnd((tokens, (hq + 2 * hkv) * d), dtype, 90, 2.0)
    positions = torch.arange(tokens, dtype=torch.int32)
    ang = torch.outer(torch.arange(64, dtype=torch.float32), 1.0 / (1e4 ** (torch.arange(0, d, 2) / d)))
    cos, sin = ang.cos().contiguous(), ang.sin().contiguous()
    kc, vc = rnd((pages, hkv, page, d), dtype, 91), rnd((pages, hkv, d, page), dtype, 92)
    kc_gpu, vc_gpu = kc.to(DEV), vc.to(DEV)
    q_gpu = torch.empty((tokens, hq, d), dtype=dtype, device=DEV)
    gpu_ops().qk_norm_rope_kv_write(qkv.to(DEV), q_gpu, kc_gpu, vc_gpu, None, None, cos.to(DEV), sin.to(DEV),
                                    positions.to(DEV), slots.to(DEV), hq, hkv, d, d, page, 1e-5)
    q_want = torch.empty((tokens, hq, d), dtype=dtype)
    PLAIN.qk_norm_rope_kv_write(qkv, q_want, kc, vc, None, None, cos, sin, positions, slots, hq, hkv, d, d, page, 1e-5)
    close(kc_gpu, kc, dtype)
    assert torch.equal(vc_gpu.cpu(), vc), "values are copied as they are, and only into their own slots"


def _attention_case(dtype, hq, hkv, d, page, window, q_lens, ctx_lens, seed, scale_one=None):
    """A batch with its cache filled at random pages; returns what both implementations need."""
    g = torch.Generator().manual_seed(seed)
    num_seqs = len(q_lens)
    order = sorted(range(num_seqs), key=lambda i: q_lens[i] == 1)
    q_lens = [q_lens[i] for i in order]
    ctx_lens = [ctx_lens[i] for i in order]
    pages_per = [-(-c // page) for c in ctx_lens]
    total_pages = sum(pages_per) + 3
    perm = torch.randperm(total_pages, generator=g).tolist()
    width = max(pages_per)
    tables = torch.zeros((num_seqs, width), dtype=torch.int32)
    at = 0
    for b, n in enumerate(pages_per):
        tables[b, :n] = torch.tensor(perm[at:at + n], dtype=torch.int32)
        at += n
    kc = (torch.randn((total_pages, hkv, page, d), generator=g)).to(dtype)
    vc = (torch.randn((total_pages, hkv, d, page), generator=g)).to(dtype)
    tokens = sum(q_lens)
    q = (torch.randn((tokens, hq, d), generator=g)).to(dtype)
    if scale_one is not None:   # make one far key stand out for one query
        b, key, boost = scale_one
        pg, off = int(tables[b, key // page]), key % page
        start = sum(q_lens[:b])
        for h in range(hq):
            kc[pg, h // (hq // hkv), off] = (q[start + q_lens[b] - 1, h].float() * boost).to(dtype)
    cu = [0]
    for n in q_lens:
        cu.append(cu[-1] + n)
    token_seq = torch.tensor([b for b, n in enumerate(q_lens) for _ in range(n)], dtype=torch.int32)
    positions = torch.tensor([ctx_lens[b] - q_lens[b] + i for b in range(num_seqs) for i in range(q_lens[b])],
                             dtype=torch.int32)
    num_prefill = sum(1 for n in q_lens if n > 1)
    rpt = 32 if max(q_lens) > 16 else 16

    def tile_list(rows):
        return torch.tensor([(b, r) for b in range(num_prefill) for r in range(0, q_lens[b], rows)] or [(0, 0)],
                            dtype=torch.int32)

    tiles = tile_list(rpt)
    tall = {rows: tile_list(rows) for rows in (32, 64, 128)} if max(q_lens) >= 32 else {}

    def meta(dev):
        return AttentionMeta(token_seq=token_seq.to(dev), positions=positions.to(dev), block_tables=tables.to(dev),
                             cu_seqlens_q=torch.tensor(cu, dtype=torch.int32).to(dev),
                             context_lens=torch.tensor(ctx_lens, dtype=torch.int32).to(dev), num_seqs=num_seqs,
                             num_tokens=tokens, max_q_len=max(q_lens), max_context_len=max(ctx_lens), page_size=page,
                             num_prefill=num_prefill, prefill_tiles=tiles.to(dev) if num_prefill else None,
                             rows_per_tile=rpt, tiles_by_rows={r: t.to(dev) for r, t in tall.items()} or None)

    return q, kc, vc, meta


ATTN_SHAPES = [  # hq, hkv, d, page
    (4, 2, 16, 16), (6, 3, 32, 8), (8, 2, 64, 16), (5, 5, 96, 4), (32, 8, 128, 16), (3, 1, 256, 32), (40, 2, 64, 16),
    (2, 1, 48, 16), (7, 7, 80, 8), (4, 2, 64, 6), (8, 2, 128, 10),   # the last two: pages no matrix-core kernel takes
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hq,hkv,d,page", ATTN_SHAPES)
@pytest.mark.parametrize("window", [None, 37])
def test_paged_attention_mixed_batch(dtype, hq, hkv, d, page, window):
    q_lens = [33, 2, 1, 1, 70, 1, 16]
    ctx_lens = [33, 150, 1, 97, 200, 310, 16]
    q, kc, vc, meta = _attention_case(dtype, hq, hkv, d, page, window, q_lens, ctx_lens, seed=hq * 100 + d)
    out = torch.empty_like(q, device=DEV)
    gpu_ops().paged_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), out, meta(DEV), d ** -0.5, window)
    want = torch.empty_like(q)
    PLAIN.paged_attention(q, kc, vc, want, meta("cpu"), d ** -0.5, window)
    close(out, want, dtype)


TILED_SHAPES = [  # hq, hkv, d, page: groups of 4, 2, 1, 3 and 8; pages of 8, 16, 32 and 64 keys
    (8, 2, 64, 16), (32, 8, 128, 16), (6, 3, 128, 8), (5, 5, 64, 32), (3, 1, 256, 8), (16, 2, 192, 64),
]


@pytest.mark.parametrize("hq,hkv,d,page", TILED_SHAPES)
@pytest.mark.parametrize("window", [None, 100])
def test_prefill_with_shared_key_tiles(hq, hkv, d, page, window):
    """Long prompt portions take the kernel whose waves share key tiles; the same batch through the
    kernel in which every wave loads its own keys, and through the plain reference."""
    ops = gpu_ops()
    assert ops.lib.atom_attention_prefill_tile_rows(d, page, hq // hkv) in (32, 64, 128)
    q_lens = [200, 33, 1, 64, 129, 1, 32]
    ctx_lens = [200, 150, 40, 500, 129, 310, 95]
    q, kc, vc, meta = _attention_case(torch.bfloat16, hq, hkv, d, page, window, q_lens, ctx_lens, seed=hq + d)
    want = torch.empty_like(q)
    PLAIN.paged_attention(q, kc, vc, want, meta("cpu"), d ** -0.5, window)
    # the kernel with shared tiles in blocks of four waves, of eight (the key tiles taken in turn by the block's
    # halves; head sizes up to 128) and of eight with 16 tokens a wave (two blocks for every listed tile, the second
    # of which may lie behind a portion's end), then the kernel whose waves load their own keys
    for tiled, halves, low in ((True, False, False), (True, True, False), (True, True, True), (False, None, None)):
        ops.use_tiled_prefill, ops.prefill_key_halves, ops.prefill_low_blocks = tiled, halves, low
        try:
            out = torch.zeros_like(q, device=DEV)
            ops.paged_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), out, meta(DEV), d ** -0.5, window)
        finally:
            ops.use_tiled_prefill, ops.prefill_key_halves, ops.prefill_low_blocks = True, None, None
        close(out, want, torch.bfloat16)


@pytest.mark.parametrize("halves,low,far", [(False, False, 300), (True, False, 300), (True, False, 364), (True, True, 300),
                                            (True, True, 364)])
def test_prefill_tiles_find_a_far_key(halves, low, far):
    """One key about 1,500 positions back, scaled so that its score stands out: the last row must return its value.
    With blocks of eight waves the key lies once in a tile of the first half (300 = 4 * 64 + 44) and once in a tile
    of the second (364 = 5 * 64 + 44), whose result reaches the output through the sum of the halves."""
    hq, hkv, d, page = 8, 2, 128, 16
    q_lens, ctx_lens = [96, 1], [1800, 5]
    q, kc, vc, meta = _attention_case(torch.bfloat16, hq, hkv, d, page, None, q_lens, ctx_lens, seed=9,
                                      scale_one=(0, far, 4.0))
    out = torch.empty_like(q, device=DEV)
    ops = gpu_ops()
    ops.prefill_key_halves, ops.prefill_low_blocks = halves, low
    try:
        ops.paged_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), out, meta(DEV), d ** -0.5, None)
    finally:
        ops.prefill_key_halves = ops.prefill_low_blocks = None
    want = torch.empty_like(q)
    PLAIN.paged_attention(q, kc, vc, want, meta("cpu"), d ** -0.5, None)
    close(out, want, torch.bfloat16)
    m = meta("cpu")
    pg, off = int(m.block_tables[0, far // page]), far % page
    for h in range(hq // hkv - 1, hq, hq // hkv):   # the key was made for the last head of each group
        got, val = out[95, h].float().cpu(), vc[pg, h // (hq // hkv), :, off].float()
        assert float((got - val).abs().max()) < 0.05 * float(val.abs().max()) + 0.05


@pytest.mark.parametrize("halves,low", [(False, False), (True, False), (True, True)])
@pytest.mark.parametrize("per_tile", [3.0, 11.0])
def test_prefill_scores_that_climb_from_tile_to_tile(per_tile, halves, low):
    """Every query's scores rise with the key's position, by `per_tile` powers of two from one tile of 64 keys to
    the next: below the step at which the tiled kernel moves a row's running maximum (so that the weights of many
    tiles are taken against an older maximum) and above it (so that it moves with every tile)."""
    hq, hkv, d, page = 8, 2, 128, 16
    q_lens, ctx_lens = [400, 1], [1400, 9]
    q, kc, vc, meta = _attention_case(torch.bfloat16, hq, hkv, d, page, None, q_lens, ctx_lens, seed=21)
    u = torch.zeros(d)
    u[5] = 1.0
    lift = 4.0
    per_key = per_tile / 64 / 1.4426950408889634 / d ** -0.5 / lift
    q = (q.float() + lift * u).to(torch.bfloat16)
    tables = meta("cpu").block_tables
    kf = kc.float()
    for key in range(ctx_lens[0]):
        kf[int(tables[0, key // page]), :, key % page] += per_key * key * u
    kc = kf.to(torch.bfloat16)
    out = torch.empty_like(q, device=DEV)
    ops = gpu_ops()
    ops.prefill_key_halves = halves    # with halves the two running maxima differ by a tile's step when they are added
    ops.prefill_low_blocks = low
    try:
        ops.paged_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), out, meta(DEV), d ** -0.5, None)
    finally:
        ops.prefill_key_halves = ops.prefill_low_blocks = None
    want = torch.empty_like(q)
    PLAIN.paged_attention(q, kc, vc, want, meta("cpu"), d ** -0.5, None)
    close(out, want, torch.bfloat16)


@pytest.mark.parametrize("parts", [1, 2, 7, 64])
@pytest.mark.parametrize("window", [None, 300])
def test_decode_split_over_waves(parts, window):
    """The decode kernel with its keys split over any number of waves, merged by the second kernel."""
    q_lens = [1, 1, 1, 1, 1]
    ctx_lens = [1, 15, 16, 700, 1025]
    q, kc, vc, meta = _attention_case(torch.bfloat16, 8, 2, 128, 16, window, q_lens, ctx_lens, seed=3)
    out = torch.empty_like(q, device=DEV)
    gpu_ops().paged_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), out, meta(DEV), 128 ** -0.5, window, parts=parts)
    want = torch.empty_like(q)
    PLAIN.paged_attention(q, kc, vc, want, meta("cpu"), 128 ** -0.5, window)
    close(out, want, torch.bfloat16)


@pytest.mark.parametrize("hq,hkv,d,page", [(6, 3, 32, 8), (16, 1, 64, 24), (40, 2, 64, 16), (3, 1, 256, 32), (4, 4, 128, 16),
                                             (5, 5, 96, 4)])
@pytest.mark.parametrize("parts", [3, 8, 9])
def test_decode_parts_in_one_block_or_merged(hq, hkv, d, page, parts):
    """Up to 8 parts of a request with up to 16 heads a KV head are the waves of one block, which merges
    them itself; more parts, larger groups and other head or page sizes go through the merge kernel."""
    q_lens = [1, 1, 1, 1]
    ctx_lens = [1, 33, 260, 1100]
    for window in (None, 200):
        q, kc, vc, meta = _attention_case(torch.bfloat16, hq, hkv, d, page, window, q_lens, ctx_lens, seed=hq + parts)
        out = torch.empty_like(q, device=DEV)
        gpu_ops().paged_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), out, meta(DEV), d ** -0.5, window, parts=parts)
        want = torch.empty_like(q)
        PLAIN.paged_attention(q, kc, vc, want, meta("cpu"), d ** -0.5, window)
        close(out, want, torch.bfloat16)


@pytest.mark.parametrize("dtype", DTYPES)
def test_far_key_among_hundreds(dtype):
    """One key far back carries nearly all the weight: an attention that drops or misplaces it
    (a wrong page, a partition edge, a tile edge) gives a visibly different output."""
    for key in (0, 15, 16, 255, 256, 511):
        q, kc, vc, meta = _attention_case(dtype, 8, 2, 64, 16, None, [40, 1], [700, 600], seed=key,
                                          scale_one=(1, key, 3.0))
        q2, kc2, vc2, meta2 = _attention_case(dtype, 8, 2, 64, 16, None, [40, 1], [700, 600], seed=key,
                                              scale_one=(0, key, 3.0))
        for (qq, kk, vv, mm) in ((q, kc, vc, meta), (q2, kc2, vc2, meta2)):
            out = torch.empty_like(qq, device=DEV)
            gpu_ops().paged_attention(qq.to(DEV), kk.to(DEV), vv.to(DEV), out, mm(DEV), 64 ** -0.5, None)
            want = torch.empty_like(qq)
            PLAIN.paged_attention(qq, kk, vv, want, mm("cpu"), 64 ** -0.5, None)
            close(out, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_far_key_in_a_long_context(dtype):
    """Contexts of 70,000 and 65,000 keys (over 4,000 pages a request, scattered over the pool): one key near the
    start carries the weight for the last row of a prompt portion and for a decode row."""
    hq, hkv, d, page = 8, 2, 128, 16
    for b, key in ((0, 1234), (1, 40001)):
        q, kc, vc, meta = _attention_case(dtype, hq, hkv, d, page, None, [64, 1], [70000, 65000], seed=b,
                                          scale_one=(b, key, 3.0))
        out = torch.empty_like(q, device=DEV)
        gpu_ops().paged_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), out, meta(DEV), d ** -0.5, None)
        want = torch.empty_like(q)
        PLAIN.paged_attention(q, kc, vc, want, meta("cpu"), d ** -0.5, None)
        close(out, want, dtype)
        row = 63 if b == 0 else 64
        m = meta("cpu")
        pg, off = int(m.block_tables[b, key // page]), key % page
        got, val = out[row, hq - 1].float().cpu(), vc[pg, hkv - 1, :, off].float()
        assert float((got - val).abs().max()) < 0.05 * float(val.abs().max()) + 0.05


def test_window_edge():
    """Keys exactly at the window's edge: position p - W + 1 is seen, p - W is not."""
    w = 40
    for dtype in DTYPES:
        for ctx in (w - 1, w, w + 1, 2 * w, 129):
            for boost_key in (ctx - w, ctx - w - 1):
                if boost_key < 0:
                    continue
                q, kc, vc, meta = _attention_case(dtype, 4, 2, 64, 16, w, [1], [ctx], seed=ctx, scale_one=(0, boost_key, 3.0))
                out = torch.empty_like(q, device=DEV)
                gpu_ops().paged_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), out, meta(DEV), 0.125, w)
                want = torch.empty_like(q)
                PLAIN.paged_attention(q, kc, vc, want, meta("cpu"), 0.125, w)
                close(out, want, dtype)


# ------------------------------------------------------------------ sampling


@pytest.mark.parametrize("vocab", [517, 151936, 20001])   # large vocabularies take the two-step argmax
def test_sample_greedy_and_ties(vocab):
    logits = rnd((9, vocab), torch.float32, 30)
    logits[3, 100] = logits[3, vocab - 117] = 50.0   # a tie, in different chunks: the lower index wins
    logits[5, vocab - 1] = 60.0
    out = torch.empty(9, dtype=torch.int32, device=DEV)
    gpu_ops().sample(logits.to(DEV), None, out)
    want = logits.argmax(dim=-1)
    want[3] = 100
    assert out.cpu().tolist() == want.tolist()


def test_noise_is_the_stated_mix():
    seeds = torch.tensor([0, 7, 2 ** 40 + 3], dtype=torch.int64)
    counters = torch.tensor([0, 5, 123456], dtype=torch.int64)
    got = gpu_ops().exponential_noise(seeds.to(DEV), counters.to(DEV), 311).cpu()
    want = torch.stack([exponential_noise_row(int(s), int(c), 311) for s, c in zip(seeds, counters)])
    assert torch.allclose(got, want, rtol=2e-6, atol=1e-7)
    big = gpu_ops().exponential_noise(torch.arange(64, dtype=torch.int64, device=DEV),
                                      torch.zeros(64, dtype=torch.int64, device=DEV), 4096)
    assert abs(float(big.mean()) - 1.0) < 0.01 and abs(float(big.var()) - 1.0) < 0.03


@pytest.mark.parametrize("top_k,top_p", [(-1, 1.0), (5, 1.0), (-1, 0.6), (20, 0.9), (1, 1.0)])
def test_sample_matches_plain_given_noise(top_k, top_p):
    rows, vocab = 12, 311
    logits = rnd((rows, vocab), torch.float32, 31, 2.0)
    temps = torch.tensor([0.7, 1.0, 0.0, 1.3] * 3, dtype=torch.float32)
    noise = torch.empty((rows, vocab)).exponential_(generator=torch.Generator().manual_seed(32))
    ks = torch.full((rows,), top_k, dtype=torch.int32)
    ps = torch.full((rows,), top_p, dtype=torch.float32)
    out = torch.empty(rows, dtype=torch.int32, device=DEV)
    gpu_ops().sample(logits.to(DEV), temps.to(DEV), out, top_ks=ks.to(DEV), top_ps=ps.to(DEV), noise=noise.to(DEV))
    want = torch.empty(rows, dtype=torch.int32)
    PLAIN.sample(logits, temps, want, top_ks=ks, top_ps=ps, noise=noise)
    assert out.cpu().tolist() == want.tolist()
    if top_k == 1:
        assert out.cpu().tolist() == logits.argmax(dim=-1).tolist()


@pytest.mark.parametrize("top_k,top_p", [(-1, 1.0), (50, 1.0), (-1, 0.8), (40, 0.95)])
def test_sample_at_a_real_vocabulary(top_k, top_p):
    """151,936 tokens: the filters and the race pick what the plain implementation picks."""
    rows, vocab = 5, 151936
    logits = rnd((rows, vocab), torch.float32, 41, 3.0)
    temps = torch.tensor([0.7, 1.0, 0.0, 1.3, 0.6], dtype=torch.float32)
    noise = torch.empty((rows, vocab)).exponential_(generator=torch.Generator().manual_seed(42))
    ks = torch.full((rows,), top_k, dtype=torch.int32)
    ps = torch.full((rows,), top_p, dtype=torch.float32)
    out = torch.empty(rows, dtype=torch.int32, device=DEV)
    gpu_ops().sample(logits.to(DEV), temps.to(DEV), out, top_ks=ks.to(DEV), top_ps=ps.to(DEV), noise=noise.to(DEV))
    want = torch.empty(rows, dtype=torch.int32)
    PLAIN.sample(logits, temps, want, top_ks=ks, top_ps=ps, noise=noise)
    assert out.cpu().tolist() == want.tolist()


def test_sample_rows_with_different_filters_at_a_real_vocabulary():
    """Rows of one call with their own temperature, top-k and top-p (off, 1, larger than the vocabulary, a p that
    keeps the likeliest token only, greedy rows between); called three times, because the kernels' histograms
    must be left empty for the next call."""
    rows, vocab = 7, 151936
    temps = torch.tensor([0.7, 1.0, 0.0, 1.3, 0.6, 0.9, 0.0], dtype=torch.float32)
    ks = torch.tensor([-1, 1, 50, 200000, 7, -1, -1], dtype=torch.int32)
    ps = torch.tensor([0.5, 1.0, 0.4, 0.9, 1.0, 1e-4, 0.3], dtype=torch.float32)
    for call in range(3):
        logits = rnd((rows, vocab), torch.float32, 50 + call, 2.0 + call)
        noise = torch.empty((rows, vocab)).exponential_(generator=torch.Generator().manual_seed(60 + call))
        out = torch.empty(rows, dtype=torch.int32, device=DEV)
        gpu_ops().sample(logits.to(DEV), temps.to(DEV), out, top_ks=ks.to(DEV), top_ps=ps.to(DEV), noise=noise.to(DEV))
        want = torch.empty(rows, dtype=torch.int32)
        PLAIN.sample(logits, temps, want, top_ks=ks, top_ps=ps, noise=noise)
        assert out.cpu().tolist() == want.tolist(), call
        assert int(out[1]) == int(logits[1].argmax()) and int(out[5]) == int(logits[5].argmax())


def test_sample_frequencies_follow_softmax():
    vocab, draws = 11, 20000
    logits = torch.tensor([[2.0, 1.0, 0.5, 0.0, -1.0, 1.5, 0.2, -3.0, 0.9, 1.1, -0.5]])
    temp = 0.7
    rep = logits.repeat(draws, 1).to(DEV)
    out = torch.empty(draws, dtype=torch.int32, device=DEV)
    gpu_ops().sample(rep, torch.full((draws,), temp, device=DEV), out,
                     seeds=torch.full((draws,), 1234, dtype=torch.int64, device=DEV),
                     counters=torch.arange(draws, dtype=torch.int64, device=DEV))
    freq = torch.bincount(out.cpu().long(), minlength=vocab).double() / draws
    want = torch.softmax(logits[0].double() / temp, dim=-1)
    assert float((freq - want).abs().max()) < 4 * math.sqrt(0.25 / draws)


def test_sample_does_not_depend_on_batch():
    logits = rnd((6, 517), torch.float32, 33, 2.0).to(DEV)
    temps = torch.full((6,), 0.8, device=DEV)
    seeds = torch.tensor([5, 6, 7, 8, 9, 10], dtype=torch.int64, device=DEV)
    counters = torch.tensor([0, 3, 1, 4, 1, 5], dtype=torch.int64, device=DEV)
    out = torch.empty(6, dtype=torch.int32, device=DEV)
    gpu_ops().sample(logits, temps, out, seeds=seeds, counters=counters)
    for r in (0, 2, 5):
        one = torch.empty(1, dtype=torch.int32, device=DEV)
        gpu_ops().sample(logits[r:r + 1].contiguous(), temps[r:r + 1].contiguous(), one,
                         seeds=seeds[r:r + 1].contiguous(), counters=counters[r:r + 1].contiguous())
        assert int(one) == int(out[r])


def test_kernels_refuse_what_they_cannot_take():
    ops = gpu_ops()
    x = torch.zeros((4, 64), device=DEV)
    with pytest.raises(KernelError):
        ops.rmsnorm(x, torch.ones(63, device=DEV), 1e-6, torch.empty_like(x))
    with pytest.raises(KernelError):
        ops.rmsnorm(x.cpu(), torch.ones(64), 1e-6, torch.empty_like(x.cpu()))
    with pytest.raises(KernelError):
        # an odd width goes through LDS, which holds 16 K floats
        ops.rmsnorm(torch.zeros((2, 20001), device=DEV), torch.ones(20001, device=DEV), 1e-6,
                    torch.zeros((2, 20001), device=DEV))
    with pytest.raises(KernelError):
        ops.silu_mul(torch.zeros((2, 7), device=DEV), torch.zeros((2, 3), device=DEV))
    with pytest.raises(KernelError):
        ops.linear(x, torch.zeros((5, 63), device=DEV))
    with pytest.raises(KernelError):
        ops.embedding(torch.zeros((10, 8), device=DEV, dtype=torch.float16), torch.zeros(2, dtype=torch.int32, device=DEV),
                      torch.zeros((2, 8), device=DEV))


# ------------------------------------------------------------------ the skinny matrix product


@pytest.fixture
def all_rows():
    """The skinny kernels for every row count they take."""
    ops = gpu_ops()
    before = ops.skinny_max_rows
    ops.skinny_max_rows = 128
    ops.use_tile_gemm = False      # (which would take the products of 65 rows and more first)
    yield ops
    ops.skinny_max_rows = before
    ops.use_tile_gemm = True


@pytest.mark.parametrize("m,n,k", [(1, 311, 136), (8, 4096, 4096), (16, 517, 200), (17, 1000, 520), (33, 96, 2056),
                                   (64, 640, 1032), (5, 64, 8), (3, 6144, 4096), (7, 130, 12288),
                                   (3, 16400, 520), (40, 16390, 1032), (8, 20000, 4096), (64, 16384, 2056),
                                   (20, 32768, 264), (50, 28672, 136), (30, 24570, 520),
                                   (18, 3, 8), (64, 7, 40), (47, 130, 12288), (17, 4098, 4096),
                                   (65, 96, 2056), (100, 640, 1032), (128, 4096, 4096), (97, 130, 12288), (81, 5, 8)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_skinny_gemm(m, n, k, out_dtype, all_rows):
    ops = all_rows
    x = rnd((m, k), torch.bfloat16, 40, 1.0)
    w = rnd((n, k), torch.bfloat16, 41, 0.05)
    b = rnd((n,), torch.float32, 42, 0.5)
    assert ops.lib.atom_gemm_skinny_supports(m, n, k)
    assert ops._skinny(x.to(DEV), w.to(DEV)), "this product must take the skinny kernel"
    want = x.double() @ w.double().T + b.double()
    y = ops.linear(x.to(DEV), w.to(DEV), b.to(DEV), out_dtype=out_dtype)
    assert y.dtype == out_dtype
    close(y, want, out_dtype if out_dtype == torch.bfloat16 else torch.bfloat16, scale=float(want.abs().max()))
    if out_dtype == torch.float32:   # float32 out keeps the float32 accumulation: far closer than a bfloat16 ulp
        assert float((y.cpu().double() - want).abs().max()) <= 1e-4 * float(want.abs().max())
    # a row's result does not depend on the rows beside it: to the bit while K is cut the same way (narrow
    # products), within rounding for the wide ones, whose blocks take what K their x slice leaves room for
    if m > 1:
        alone = ops.linear(x[m - 1:].to(DEV).contiguous(), w.to(DEV), b.to(DEV), out_dtype=out_dtype)
        if n < 256 * 64 and m <= 8:
            assert torch.equal(alone[0], y[m - 1])
        else:
            close(alone[0], y[m - 1].double(), torch.bfloat16)
    if m > 9:   # more than 8 rows: another kernel, whose cut of K does not depend on the row count
        fewer = ops.linear(x[m - 9:].to(DEV).contiguous(), w.to(DEV), b.to(DEV), out_dtype=out_dtype)
        assert torch.equal(fewer[8], y[m - 1])


@pytest.mark.parametrize("m,n,k", [(65, 4096, 4096), (96, 2560, 9728), (128, 6144, 2560), (200, 130, 12288),
                                   (256, 5120, 5120), (129, 517, 1024), (255, 4096, 12288), (70, 7, 64),
                                   (100, 1031, 192), (256, 8192, 576)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_tile_gemm(m, n, k, out_dtype):
    """65 to 256 rows: the kernel of tiles and K slices cut to the chip, at the widths of the 4B, 8B and 32B shapes
    and at sizes that are no multiple of anything: against the float64 product, whole or left as a sum of slices."""
    from atom_amd.kernels.hip import DeferredSum

    ops = gpu_ops()
    x = rnd((m, k), torch.bfloat16, 60, 1.0)
    w = rnd((n, k), torch.bfloat16, 61, 0.05)
    b = rnd((n,), torch.float32, 62, 0.5)
    assert ops._tile(x.to(DEV), w.to(DEV)), "this product must take the tile kernel"
    want = x.double() @ w.double().T + b.double()
    ops.allow_library_gemm = False
    try:
        y = ops.linear(x.to(DEV), w.to(DEV), b.to(DEV), out_dtype=out_dtype)
        lazy = ops.linear(x.to(DEV), w.to(DEV), b.to(DEV), out_dtype=out_dtype, defer=True)
    finally:
        ops.allow_library_gemm = True
    assert y.dtype == out_dtype
    close(y, want, torch.bfloat16, scale=float(want.abs().max()))
    if out_dtype == torch.float32:
        assert float((y.cpu().double() - want).abs().max()) <= 1e-4 * float(want.abs().max())
    splits = ops.lib.atom_gemm_tile_splits(m, n, k, ops.num_cus)
    if splits > 1 and n <= k:    # a sum of slices for the norm behind it to add
        assert isinstance(lazy, DeferredSum) and lazy.splits == splits
        total = lazy.partial.double().sum(0).cpu() + b.double()
        assert float((total - want).abs().max()) <= 1e-4 * float(want.abs().max())
        assert torch.equal(ops.materialize(lazy), y)
    else:
        assert torch.equal(lazy, y)
    # a row's result does not depend on how many rows stand beside it, as long as the tile kernel runs (the
    # slices of K depend on the number of tiles, so across a tile's edge only within rounding)
    fewer = ops.linear(x[m - 65:].to(DEV).contiguous(), w.to(DEV), b.to(DEV), out_dtype=out_dtype)
    close(fewer[64], y[m - 1].double(), torch.bfloat16, scale=float(want.abs().max()))


def test_tile_gemm_plan():
    """The slices of K: the most that keep tiles x slices within the CUs, whole stages, eight of them at least."""
    lib = gpu_ops().lib
    assert lib.atom_gemm_tile_splits(256, 4096, 4096, 256) == 4       # 64 tiles
    assert lib.atom_gemm_tile_splits(256, 6144, 4096, 256) == 2       # 96 tiles
    assert lib.atom_gemm_tile_splits(96, 4096, 12288, 256) == 8       # 32 tiles
    assert lib.atom_gemm_tile_splits(128, 2560, 9728, 256) == 8       # 20 tiles
    assert lib.atom_gemm_tile_splits(128, 2560, 9728 - 64, 256) == 1  # 151 stages: an odd number
    assert lib.atom_gemm_tile_splits(256, 8192, 576, 256) == 1        # a slice would be shorter than eight stages
    assert lib.atom_gemm_tile_splits(256, 24576, 4096, 256) == 1      # 384 tiles fill the chip as they are
    assert lib.atom_gemm_tile_splits(100, 640, 1032, 256) == 0 and not lib.atom_gemm_tile_supports(100, 640, 1032)


def test_skinny_gemm_is_what_runs():
    """Few bfloat16 rows take the engine's own kernel, not the library."""
    ops = gpu_ops()
    x = rnd((8, 512), torch.bfloat16, 1).to(DEV)
    w = rnd((256, 512), torch.bfloat16, 2, 0.05).to(DEV)
    ops.allow_library_gemm = False
    try:
        y = ops.linear(x, w)
    finally:
        ops.allow_library_gemm = True
    close(y, x.cpu().double() @ w.cpu().double().T, torch.bfloat16)


@pytest.mark.parametrize("m,inter,k", [(1, 200, 136), (8, 12288, 4096), (20, 333, 264), (64, 160, 96),
                                       (33, 8200, 1032), (64, 8192, 4096), (24, 14336, 136), (48, 12287, 264),
                                       (17, 16384, 72), (18, 3, 8), (40, 6, 16), (64, 1001, 2056),
                                       (128, 160, 96), (70, 333, 264)])
def test_skinny_gemm_silu_gate(m, inter, k, all_rows):
    ops = all_rows
    x = rnd((m, k), torch.bfloat16, 50, 1.0)
    w = rnd((2 * inter, k), torch.bfloat16, 51, 0.05)
    b = rnd((2 * inter,), torch.float32, 52, 0.3)
    gu = x.double() @ w.double().T + b.double()
    want = torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:]
    act = ops.linear_silu(x.to(DEV), w.to(DEV), b.to(DEV))
    close(act, want, torch.bfloat16)
    swapped = torch.nn.functional.silu(gu[:, inter:]) * gu[:, :inter]
    assert float((swapped - want).abs().max()) > 0.05 * float(want.abs().max())


def _deferred(ops, m, n, k, seed, bias=True):
    """A product as the skinny kernel leaves it when it cuts K, and the same as float64."""
    from atom_amd.kernels.hip import DeferredSum

    x = rnd((m, k), torch.bfloat16, seed, 1.0)
    w = rnd((n, k), torch.bfloat16, seed + 1, 0.05)
    b = rnd((n,), torch.float32, seed + 2, 0.3) if bias else None
    ops.use_rows_gemm = False    # few rows would otherwise take the product that cuts nothing
    try:
        got = ops.linear(x.to(DEV), w.to(DEV), b.to(DEV) if bias else None, defer=True)
    finally:
        ops.use_rows_gemm = True
    assert isinstance(got, DeferredSum) and got.splits > 1, "this shape was chosen so that K is cut"
    want = x.double() @ w.double().T + (b.double() if bias else 0)
    return got, want


def test_deferred_sum_readers():
    """Norm, rotation and SiLU-mul read a product that is still a sum of slices."""
    ops = gpu_ops()
    # norm with the residual sum
    d, want = _deferred(ops, 6, 256, 4096, 60)
    wn = 1 + rnd((256,), torch.float32, 63, 0.2)
    res = rnd((6, 256), torch.float32, 64)
    out = torch.empty((6, 256), dtype=torch.bfloat16, device=DEV)
    res_gpu = res.to(DEV)
    ops.rmsnorm(d, wn.to(DEV), 1e-5, out, residual=res_gpu, mode="add")
    summed = want + res.double()
    norm = summed * torch.rsqrt((summed ** 2).mean(-1, keepdim=True) + 1e-5) * wn.double()
    close(out, norm, torch.bfloat16)
    close(res_gpu, summed, torch.float32, scale=float(summed.abs().max()) * 50)   # sums of bfloat16 products
    # norm at chosen rows, width that is no multiple of 8 pieces per thread
    rows = torch.tensor([5, 0], dtype=torch.int32, device=DEV)
    out2 = torch.empty((2, 256), dtype=torch.bfloat16, device=DEV)
    ops.rmsnorm(d, wn.to(DEV), 1e-5, out2, residual=res.to(DEV), mode="add", rows=rows)
    close(out2, norm[[5, 0]], torch.bfloat16)
    # materialize
    close(ops.materialize(d), want, torch.bfloat16)
    # SiLU-mul
    d, want = _deferred(ops, 4, 2 * 136, 2048, 70)
    act = torch.empty((4, 136), dtype=torch.bfloat16, device=DEV)
    ops.silu_mul(d, act)
    close(act, torch.nn.functional.silu(want[:, :136]) * want[:, 136:], torch.bfloat16)
    # rotation and cache write: against the same kernel fed the tensor
    hq, hkv, hd, page = 4, 2, 32, 16
    d, want = _deferred(ops, 5, (hq + 2 * hkv) * hd, 4096, 80)
    qkv = want.to(torch.bfloat16).to(DEV)
    pos = torch.tensor([3, 9, 0, 17, 30], dtype=torch.int32, device=DEV)
    slots = torch.tensor([3, 9, 16, -1, 46], dtype=torch.int32, device=DEV)
    inv = 1.0 / (10000.0 ** (torch.arange(0, hd, 2).float() / hd))
    ang = torch.arange(64).float()[:, None] * inv[None, :]
    cos, sin = ang.cos().to(DEV), ang.sin().to(DEV)
    wq = (1 + rnd((hd,), torch.float32, 83, 0.2)).to(DEV)
    wk = (1 + rnd((hd,), torch.float32, 84, 0.2)).to(DEV)
    outs = []
    for src in (d, qkv):
        q = torch.zeros((5, hq, hd), dtype=torch.bfloat16, device=DEV)
        kc = torch.zeros((4, hkv, page, hd), dtype=torch.bfloat16, device=DEV)
        vc = torch.zeros((4, hkv, hd, page), dtype=torch.bfloat16, device=DEV)
        ops.qk_norm_rope_kv_write(src, q, kc, vc, wq, wk, cos, sin, pos, slots, hq, hkv, hd, hd, page, 1e-6)
        outs.append((q, kc, vc))
    for a, b in zip(*outs):
        close(a, b.double(), torch.bfloat16, scale=float(b.abs().max()) * 2)


def test_feed_tokens():
    ops = gpu_ops()
    gen = torch.Generator().manual_seed(3)
    for n in (1, 7, 300):
        ids = torch.randint(0, 1000, (n,), generator=gen, dtype=torch.int32)
        sampled = torch.randint(1000, 2000, (9,), generator=gen, dtype=torch.int32)
        source = torch.randint(-1, 9, (n,), generator=gen, dtype=torch.int32)
        want = torch.where(source >= 0, sampled[source.clamp(min=0).long()], ids)
        got = ops.feed_tokens(ids.cuda(), source.cuda(), sampled.cuda())
        assert torch.equal(got.cpu(), want)


# ------------------------------------------------------------------ the few-rows product with norm and residual folded in


@pytest.mark.parametrize("m", [1, 2, 3, 5, 8])
@pytest.mark.parametrize("n,k", [(311, 136), (4096, 4096), (6144, 2560), (130, 12288), (16, 8), (1031, 520), (5000, 9728)])
@pytest.mark.parametrize("waves,narrow", [(0, True), (4, True), (8, True), (0, False)])
def test_rows_product_plain_gate_and_residual(m, n, k, waves, narrow):
    """(The widths take tiles of 16, 12 and 8 columns a block: 4,096 of 16, 6,144 and 5,000 of 12, the small ones
    of 8; with ``narrow`` off all take 16.)"""
    from atom_amd.kernels.hip import PendingNorm, PendingProduct

    ops = gpu_ops()
    ops.rows_waves = waves
    ops.narrow_row_tiles = narrow
    assert [ops.rows_cols(w) for w in (4096, 6144, 5000, 311, 16)] == ([16, 12, 12, 8, 8] if narrow else [16] * 5)
    ops._rows_residual_pays = lambda n, k: True   # the folded residual sum at every size, also where the split way is faster
    try:
        x = rnd((m, k), torch.bfloat16, 50, 1.0)
        w = rnd((n, k), torch.bfloat16, 51, 0.05)
        b = rnd((n,), torch.float32, 52, 0.5)
        want = x.double() @ w.double().T + b.double()
        scale = float(want.abs().max())
        assert ops._rows_takes(x.to(DEV), w.to(DEV))
        for out_dtype in (torch.bfloat16, torch.float32):
            y = ops.linear(x.to(DEV), w.to(DEV), b.to(DEV), out_dtype=out_dtype)
            assert y.dtype == out_dtype
            close(y, want, torch.bfloat16, scale=scale)
            if out_dtype == torch.float32:
                assert float((y.cpu().double() - want).abs().max()) <= 1e-4 * scale
                alone = ops.linear(x[m - 1:].to(DEV).contiguous(), w.to(DEV), b.to(DEV), out_dtype=out_dtype)
                assert torch.equal(alone[0], y[m - 1]), "a row's sum does not depend on the rows beside it"
        # deferred: nothing is launched until something wants it
        pending = ops.linear(x.to(DEV), w.to(DEV), b.to(DEV), defer=True)
        assert isinstance(pending, PendingProduct) and tuple(pending.shape) == (m, n)
        close(ops.materialize(pending), want, torch.bfloat16, scale=scale)
        # ... a norm with the residual stream makes it add in place and leaves the norm pending
        res = rnd((m, n), torch.float32, 53, 2.0)
        gamma = 1 + rnd((n,), torch.float32, 54, 0.2)
        res_gpu = res.to(DEV)
        lazy = ops.pending_norm(pending, res_gpu, gamma.to(DEV), 1e-5)
        assert isinstance(lazy, PendingNorm) and lazy.r is res_gpu
        new_res = res.double() + want
        assert float((res_gpu.cpu().double() - new_res).abs().max()) <= 1e-4 * float(new_res.abs().max())
        ss_want = new_res.pow(2).sum(-1)
        assert torch.allclose(lazy.ss.sum(-1).cpu().double(), ss_want, rtol=1e-5)
        normed_want = new_res * torch.rsqrt(new_res.pow(2).mean(-1, keepdim=True) + 1e-5) * gamma.double()
        close(ops.materialize(lazy), normed_want, torch.bfloat16)
        # ... which the next product applies while it reads (here: back down to a width of 200, and SiLU-gated)
        if n % 8 == 0:
            w2 = rnd((200, n), torch.bfloat16, 55, 0.05)
            xn = normed_want.to(torch.bfloat16).double()
            y2 = ops.linear(lazy, w2.to(DEV), None, out_dtype=torch.float32)
            want2 = xn @ w2.double().T
            assert float((y2.cpu().double() - want2).abs().max()) <= 1.2e-2 * float(want2.abs().max())
            wg = rnd((2 * 104, n), torch.bfloat16, 56, 0.05)
            bg = rnd((2 * 104,), torch.float32, 57, 0.3)
            act = ops.linear_silu(lazy, wg.to(DEV), bg.to(DEV))
            gu = xn @ wg.double().T + bg.double()
            want_act = torch.nn.functional.silu(gu[:, :104]) * gu[:, 104:]
            close(act, want_act, torch.bfloat16)
            # ... also at chosen rows only (the head of a step that wants some rows' logits)
            if m >= 3:
                pick = torch.tensor([m - 1, 0], dtype=torch.int32, device=DEV)
                picked = PendingNorm(lazy.r, lazy.xg, lazy.ss, lazy.weight, lazy.eps, pick, lazy.dtype)
                y3 = ops.linear(picked, w2.to(DEV), None, out_dtype=torch.float32)
                assert torch.equal(y3[0], y2[m - 1]) and torch.equal(y3[1], y2[0])
    finally:
        ops.rows_waves = 0
        ops.narrow_row_tiles = True
        del ops._rows_residual_pays


def test_row_tiles_narrow_where_that_spreads_the_columns():
    """Tiles of 12 or 8 columns where they take a fifth off the busiest CU's columns (256 CUs): the 4B width (160
    tiles of 16) and the widths of 1.25 and 1.5 tiles of 16 a CU; not the 8B width, the vocabulary or gate/up."""
    ops = gpu_ops()
    assert ops.num_cus == 256
    assert [ops.rows_cols(n) for n in (2560, 5120, 6144, 3072, 1024)] == [12, 12, 12, 12, 8]
    assert [ops.rows_cols(n) for n in (4096, 8192, 10240, 151936, 24576, 3584)] == [16] * 6
    assert ops.lib.atom_gemm_rows_parts(2560, 12) == 214 and ops.lib.atom_gemm_rows_parts(2560, 16) == 160
    assert ops.lib.atom_gemm_rows_parts(2560, 10) == 0


def test_residual_product_with_too_few_tiles_goes_the_split_way():
    """A product of 160 column tiles and a long K (135 MB of weights): the few-rows kernel with the residual sum
    folded in would leave 96 CUs idle, so the norm launches the product with K cut between blocks and adds the
    slices itself; the same numbers come out."""
    from atom_amd.kernels.hip import DeferredSum, PendingProduct

    ops = gpu_ops()
    m, n, k = 5, 2560, 26400
    assert all(ops._rows_residual_pays(*nk) for nk in [(4096, 12288), (4096, 4096), (2560, 9728), (2560, 4096), (5120, 8192),
                                                       (5120, 25600), (n, k)])
    ops.narrow_row_tiles = False     # with tiles of 16 columns only, these two leave CUs idle for too long
    try:
        assert not ops._rows_residual_pays(n, k) and not ops._rows_residual_pays(5120, 25600)
        assert all(ops._rows_residual_pays(*nk) for nk in [(4096, 12288), (4096, 4096), (2560, 9728), (2560, 4096), (5120, 8192)])
        x = rnd((m, k), torch.bfloat16, 70, 1.0)
        w = rnd((n, k), torch.bfloat16, 71, 0.02)
        want = x.double() @ w.double().T
        res = rnd((m, n), torch.float32, 72, 2.0)
        gamma = 1 + rnd((n,), torch.float32, 73, 0.2)
        pending = ops.linear(x.to(DEV), w.to(DEV), None, defer=True)
        assert isinstance(pending, PendingProduct)
        res_gpu = res.to(DEV)
        assert ops.pending_norm(pending, res_gpu, gamma.to(DEV), 1e-6) is None and pending.split
        assert isinstance(ops.linear(x.to(DEV), w.to(DEV), None, defer=True, few_rows=False), DeferredSum)
        out = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
        ops.rmsnorm(pending, gamma.to(DEV), 1e-6, out, residual=res_gpu, mode="add")
        new_res = res.double() + want
        assert float((res_gpu.cpu().double() - new_res).abs().max()) <= 1e-4 * float(new_res.abs().max())
        close(out, new_res * torch.rsqrt(new_res.pow(2).mean(-1, keepdim=True) + 1e-6) * gamma.double(), torch.bfloat16)
    finally:
        ops.narrow_row_tiles = True


@pytest.mark.parametrize("n,k", [(2560, 4096), (2560, 9728), (5120, 8192), (5120, 25600)])
def test_residual_product_both_ways_at_the_4b_and_32b_widths(n, k):
    """The o and down products of the 4B and 32B shapes with the residual sum folded in and with K cut between blocks
    plus the add-norm kernel, whichever of the two the chip's figures choose: both give the reference's residual
    stream and norm, so the choice changes speed and the last bits only."""
    from atom_amd.kernels.hip import PendingNorm, PendingProduct

    ops = gpu_ops()
    m = 6
    x = rnd((m, k), torch.bfloat16, 80, 1.0)
    w = rnd((n, k), torch.bfloat16, 81, 0.02)
    res = rnd((m, n), torch.float32, 82, 2.0)
    gamma = 1 + rnd((n,), torch.float32, 83, 0.2)
    new_res = res.double() + x.double() @ w.double().T
    normed = new_res * torch.rsqrt(new_res.pow(2).mean(-1, keepdim=True) + 1e-6) * gamma.double()
    chosen = ops._rows_residual_pays(n, k)
    for folded in (True, False):
        ops._rows_residual_pays = lambda n_, k_, f=folded: f
        try:
            pending = ops.linear(x.to(DEV), w.to(DEV), None, defer=True)
            assert isinstance(pending, PendingProduct)
            res_gpu = res.to(DEV)
            lazy = ops.pending_norm(pending, res_gpu, gamma.to(DEV), 1e-6)
            if folded:
                assert isinstance(lazy, PendingNorm)
                out = ops.materialize(lazy)
            else:
                assert lazy is None and pending.split
                out = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
                ops.rmsnorm(pending, gamma.to(DEV), 1e-6, out, residual=res_gpu, mode="add")
        finally:
            del ops._rows_residual_pays
        assert float((res_gpu.cpu().double() - new_res).abs().max()) <= 1e-4 * float(new_res.abs().max()), (folded, chosen)
        close(out, normed, torch.bfloat16)


def test_rows_product_gate_alone_and_odd_widths():
    ops = gpu_ops()
    for m, inter, k in [(1, 200, 136), (8, 12288, 4096), (4, 333, 264), (7, 9, 40)]:
        x = rnd((m, k), torch.bfloat16, 60, 1.0)
        w = rnd((2 * inter, k), torch.bfloat16, 61, 0.05)
        b = rnd((2 * inter,), torch.float32, 62, 0.3)
        gu = x.double() @ w.double().T + b.double()
        want = torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:]
        close(ops.linear_silu(x.to(DEV), w.to(DEV), b.to(DEV)), want, torch.bfloat16)


# ------------------------------------------------------------------ decode attention that starts from the QKV product


@pytest.mark.parametrize("hq,hkv,d,page", [(32, 8, 128, 16), (8, 2, 64, 8), (6, 3, 64, 16), (4, 1, 256, 32), (40, 2, 128, 16)])
@pytest.mark.parametrize("norm", [True, False])
@pytest.mark.parametrize("window", [None, 40])
def test_fused_decode_attention_matches_the_separate_kernels(hq, hkv, d, page, norm, window):
    """Per-head norm, rotation, cache write and attention in one kernel against the same step as two kernels,
    for requests whose new token is the first of a page, the last, in the middle, and a padding row."""
    from atom_amd.kernels.hip import PendingProduct

    ops = gpu_ops()
    ctxs = [1, page, page + 1, 5 * page - 1, 333, 0, 97]       # keys of each request with the new token; 0: padding
    seqs, hidden = len(ctxs), 264
    width = -(-max(ctxs) // page)
    pages = seqs * width + 1
    g = torch.Generator().manual_seed(7)
    tables = torch.randperm(pages - 1, generator=g)[:seqs * width].view(seqs, width).to(torch.int32) + 1
    x = rnd((seqs, hidden), torch.bfloat16, 90)
    w = rnd(((hq + 2 * hkv) * d, hidden), torch.bfloat16, 91, 0.1)
    b = rnd(((hq + 2 * hkv) * d,), torch.float32, 92, 0.3)
    qw = (1 + rnd((d,), torch.float32, 93, 0.2)).to(DEV) if norm else None
    kw = (1 + rnd((d,), torch.float32, 94, 0.2)).to(DEV) if norm else None
    inv = 1.0 / (10000.0 ** (torch.arange(0, d, 2).float() / d))
    ang = torch.arange(512).float()[:, None] * inv[None, :]
    cos, sin = ang.cos().to(DEV), ang.sin().to(DEV)
    k0 = rnd((pages, hkv, page, d), torch.bfloat16, 95)
    v0 = rnd((pages, hkv, d, page), torch.bfloat16, 96)
    pos = torch.tensor([max(c - 1, 0) for c in ctxs], dtype=torch.int32)
    slots = torch.tensor([int(tables[s, (c - 1) // page]) * page + (c - 1) % page if c else -1 for s, c in enumerate(ctxs)],
                         dtype=torch.int32)
    meta = AttentionMeta(token_seq=torch.tensor([s if c else -1 for s, c in enumerate(ctxs)], dtype=torch.int32).to(DEV),
                         positions=pos.to(DEV), block_tables=tables.to(DEV).contiguous(),
                         cu_seqlens_q=torch.arange(seqs + 1, dtype=torch.int32).to(DEV),
                         context_lens=torch.tensor(ctxs, dtype=torch.int32).to(DEV), num_seqs=seqs, num_tokens=seqs,
                         max_q_len=1, max_context_len=max(ctxs), page_size=page, num_prefill=0)

    def pending():
        got = ops.linear(x.to(DEV), w.to(DEV), b.to(DEV), defer=True)
        assert isinstance(got, PendingProduct)
        return got

    results = []
    for fused in (True, False):
        kc, vc = k0.clone().to(DEV), v0.clone().to(DEV)
        out = torch.full((seqs, hq, d), float("nan"), dtype=torch.bfloat16, device=DEV)
        for parts in (1, 4, 13):
            if fused:
                done = ops.fused_decode_attention(pending(), kc, vc, out, meta, d ** -0.5, window, qw, kw, cos, sin,
                                                  slots.to(DEV), hq, hkv, d, d, 1e-5, parts=parts)
                assert done is out
            else:
                q = torch.empty((seqs, hq, d), dtype=torch.bfloat16, device=DEV)
                ops.qk_norm_rope_kv_write(pending(), q, kc, vc, qw, kw, cos, sin, pos.to(DEV), slots.to(DEV), hq, hkv, d, d,
                                          page, 1e-5)
                ops.paged_attention(q, kc, vc, out, meta, d ** -0.5, window, parts=parts)
            results.append((fused, parts, out.clone().cpu(), kc.cpu().clone(), vc.cpu().clone()))
    want = {parts: r for f, parts, *r in results if not f}
    for f, parts, out, kc, vc in results:
        if not f:
            continue
        ref_out, ref_k, ref_v = want[parts]
        assert torch.equal(vc, ref_v), "the new values land in the same places"
        assert float((kc.float() - ref_k.float()).abs().max()) <= 2e-2 * float(ref_k.float().abs().max())
        assert (kc != ref_k).float().mean() < 1e-3, "only the new keys may differ, and only by a rounding"
        live = [s for s, c in enumerate(ctxs) if c]
        close(out[live], ref_out[live].double(), torch.bfloat16)
        assert float(out[ctxs.index(0)].float().abs().max()) == 0.0, "a padding row attends to nothing"
    # a layer that reads another layer's cache writes nothing
    kc, vc = k0.clone().to(DEV), v0.clone().to(DEV)
    out = torch.empty((seqs, hq, d), dtype=torch.bfloat16, device=DEV)
    ops.fused_decode_attention(pending(), kc, vc, out, meta, d ** -0.5, window, qw, kw, cos, sin, None, hq, hkv, d, d,
                               1e-5, write_kv=False)
    assert torch.equal(kc.cpu(), k0) and torch.equal(vc.cpu(), v0)
