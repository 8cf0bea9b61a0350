"""Each HIP kernel alone against its plain torch reference (tests/torch_ops.py), at sizes other
than the engine's tiny models: head sizes in steps of 16, odd numbers of heads and groups,
widths and vocabularies that are no power of two, float32 and bfloat16."""
import math

import pytest
import torch

from torch_ops import TorchOps

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from lmsf_amd.ops import get_ops
    return get_ops()


@pytest.fixture(scope="module")
def ref():
    return TorchOps()


def dev(t):
    return t.to("cuda:0")


def tol(dtype):
    return dict(atol=2e-5, rtol=2e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


def test_library_is_loaded(ops):
    from lmsf_amd.ops import library_path
    assert library_path() and library_path().endswith("liblmsf_hip.so")
    assert ops.device_arch.startswith("gfx950")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("V,H,N", [(331, 80, 7), (1000, 4096, 33), (50, 17, 1)])
def test_embedding(ops, ref, dtype, V, H, N):
    g = torch.Generator().manual_seed(V + H)
    table = dev(torch.randn(V, H, generator=g).to(dtype))
    ids = dev(torch.randint(0, V, (N,), generator=g, dtype=torch.int32))
    out = ops.embedding(ids, table, 1.5)
    assert out.dtype == torch.float32
    assert torch.equal(out, ref.embedding(ids, table, 1.5))


def test_embedding_flags_bad_id(ops):
    table = dev(torch.randn(10, 8))
    out = ops.embedding(dev(torch.tensor([3, 11, -1], dtype=torch.int32)), table)
    assert ops.bad_token_seen()
    assert not ops.bad_token_seen()
    assert torch.equal(out[1], torch.zeros(8, device="cuda:0")) and torch.equal(out[0], table[3])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N,H", [(5, 80), (3, 4096), (2, 5000), (9, 17)])
def test_add_rms_norm(ops, ref, dtype, N, H):
    g = torch.Generator().manual_seed(N * H)
    branch = dev((torch.randn(N, H, generator=g) * 3).to(dtype))
    res = dev(torch.randn(N, H, generator=g))
    w = dev(torch.randn(H, generator=g).to(dtype))
    for eps, off in ((1e-5, 0.0), (1e-6, 1.0)):
        r1, r2 = res.clone(), res.clone()
        a = ops.add_rms_norm(branch, r1, w, eps, dtype, weight_offset=off)
        b = ref.add_rms_norm(branch, r2, w, eps, dtype, weight_offset=off)
        assert torch.allclose(r1, r2, atol=1e-6, rtol=1e-6)
        assert torch.allclose(a.float(), b.float(), **tol(dtype))
    # norm of the stream alone, of a branch alone, and gathered rows
    a = ops.add_rms_norm(None, res.clone(), w, 1e-5, dtype)
    assert torch.allclose(a.float(), ref.add_rms_norm(None, res.clone(), w, 1e-5, dtype).float(), **tol(dtype))
    a = ops.add_rms_norm(branch, None, w, 1e-5, dtype)
    assert torch.allclose(a.float(), ref.add_rms_norm(branch, None, w, 1e-5, dtype).float(), **tol(dtype))
    rows = dev(torch.tensor([N - 1, 0], dtype=torch.int32))
    r1 = res.clone()
    a = ops.add_rms_norm(branch, r1, w, 1e-5, dtype, rows=rows)
    assert torch.equal(r1, res)          # a gather leaves the stream alone
    assert torch.allclose(a.float(), ref.add_rms_norm(branch, res.clone(), w, 1e-5, dtype, rows=rows).float(),
                          **tol(dtype))
    # float32 weight with bfloat16 activations
    if dtype == torch.bfloat16:
        a = ops.add_rms_norm(branch, res.clone(), w.float(), 1e-5, dtype)
        assert torch.allclose(a.float(), ref.add_rms_norm(branch, res.clone(), w.float(), 1e-5, dtype).float(),
                              **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,rot,neox,ps", [(5, 5, 48, 48, True, 16), (6, 2, 64, 32, False, 8),
                                                 (8, 1, 128, 128, True, 16), (3, 3, 16, 16, True, 4)])
@pytest.mark.parametrize("N", [11, 150])
def test_rope_cache_write(ops, ref, dtype, nh, nkv, d, rot, neox, ps, N):
    """N = 150: the kernel for steps of many tokens (tiles of 16 tokens, 16-byte pieces) where the sizes
    allow it; slots partly in runs (a prompt's portion), partly scattered."""
    g = torch.Generator().manual_seed(nh * d)
    max_pos, pages = 64, -(-N // ps) + 6
    qkv = dev(torch.randn(N, (nh + 2 * nkv) * d, generator=g).to(dtype))
    pos = dev(torch.randint(0, max_pos, (N,), generator=g, dtype=torch.int32))
    ang = torch.arange(max_pos, dtype=torch.float32)[:, None] * torch.rand(rot // 2, generator=g)[None, :]
    table = dev(torch.cat([ang.cos(), ang.sin()], dim=1).contiguous())
    slots = torch.randperm(pages * ps, generator=g)[:N].to(torch.int32)
    if N > 64:
        run = torch.arange(5, 5 + 100, dtype=torch.int32)          # 100 consecutive slots from an odd start
        rest = torch.tensor([s for s in slots.tolist() if s < 5 or s >= 105][:N - 100], dtype=torch.int32)
        slots = torch.cat([rest[:7], run, rest[7:]])
        assert slots.numel() == N and len(set(slots.tolist())) == N
    slots[3] = -1
    slots = dev(slots)
    k1, v1 = dev(torch.zeros((pages, nkv, ps, d), dtype=dtype)), dev(torch.zeros((pages, nkv, d, ps), dtype=dtype))
    k2, v2 = k1.clone(), v1.clone()
    a, b = qkv.clone(), qkv.clone()
    ops.rope_cache_write(a, nh, nkv, d, pos, table, rot, neox, slots, k1, v1)
    ref.rope_cache_write(b, nh, nkv, d, pos, table, rot, neox, slots, k2, v2)
    assert torch.allclose(a.float(), b.float(), **tol(dtype))
    assert torch.allclose(k1.float(), k2.float(), **tol(dtype)) and torch.equal(v1, v2)
    # cache write alone and rotation alone
    a, b = qkv.clone(), qkv.clone()
    k1.zero_(); v1.zero_(); k2.zero_(); v2.zero_()
    ops.rope_cache_write(a, nh, nkv, d, None, None, 0, True, slots, k1, v1)
    ref.rope_cache_write(b, nh, nkv, d, None, None, 0, True, slots, k2, v2)
    assert torch.equal(a, qkv) and torch.equal(k1, k2) and torch.equal(v1, v2)
    ops.rope_cache_write(a, nh, nkv, d, pos, table, rot, neox, None, None, None)
    ref.rope_cache_write(b, nh, nkv, d, pos, table, rot, neox, None, None, None)
    assert torch.allclose(a.float(), b.float(), **tol(dtype))


def _paged_case(dtype, nh, nkv, d, ps, seg_lens, ctx_lens, seed, spike=False):
    """Segments with ``seg_lens`` query tokens each at the end of contexts of ``ctx_lens`` tokens; pages in
    a scrambled order. Returns the kernel's arguments."""
    g = torch.Generator().manual_seed(seed)
    S = len(seg_lens)
    blocks = [-(-c // ps) for c in ctx_lens]
    total = sum(blocks) + 3
    perm = torch.randperm(total, generator=g).tolist()
    W = max(blocks)
    bt = torch.zeros(S, W, dtype=torch.int32)
    at = 0
    for s in range(S):
        for b in range(blocks[s]):
            bt[s, b] = perm[at]
            at += 1
    k_pages = torch.randn(total, nkv, ps, d, generator=g)
    v_pages = torch.randn(total, nkv, d, ps, generator=g)
    N = sum(seg_lens)
    q = torch.randn(N, nh * d + 8, generator=g)       # wider than nh*d: a strided view, like the fused QKV
    seg, pos = [], []
    for s in range(S):
        for i in range(seg_lens[s]):
            seg.append(s)
            pos.append(ctx_lens[s] - seg_lens[s] + i)
    if spike:
        # one far key per kv head stands out: scale it and the matching query direction
        for s in range(S):
            j = 1 if ctx_lens[s] > 1 else 0
            page, off = int(bt[s, j // ps]), j % ps
            k_pages[page, :, off, :] *= 6.0
    return (dev(q.to(dtype)), dev(k_pages.to(dtype)), dev(v_pages.to(dtype)), dev(bt),
            dev(torch.tensor(seg, dtype=torch.int32)), dev(torch.tensor(pos, dtype=torch.int32)))


ATT_SHAPES = [
    # nh, nkv, d, page size, query tokens per segment, context per segment
    (4, 2, 16, 8, [1, 7, 33], [1, 7, 33]),
    (5, 5, 48, 16, [2, 1, 1], [300, 17, 256]),
    (8, 1, 32, 16, [64, 1], [64, 513]),
    (6, 3, 80, 4, [3, 5], [40, 5]),
    (32, 8, 128, 16, [1, 1, 1, 16], [700, 1, 257, 16]),
    (2, 1, 256, 32, [9], [70]),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", ATT_SHAPES)
@pytest.mark.parametrize("window", [0, 24])
def test_paged_attention(ops, ref, dtype, shape, window):
    nh, nkv, d, ps, seg_lens, ctx_lens = shape
    q, kp, vp, bt, seg, pos = _paged_case(dtype, nh, nkv, d, ps, seg_lens, ctx_lens, seed=nh * d + ps, spike=True)
    scale = 1.0 / math.sqrt(d)
    a = ops.paged_attention(q, kp, vp, bt, seg, pos, nh, nkv, d, scale, window)
    b = ref.paged_attention(q, kp, vp, bt, seg, pos, nh, nkv, d, scale, window)
    assert a.shape == (q.shape[0], nh * d)
    assert torch.allclose(a.float(), b.float(), **tol(dtype)), (a.float() - b.float()).abs().max()


MFMA_SHAPES = [
    # nh, nkv, d, page size, query tokens per segment, context per segment
    (4, 2, 16, 8, [1, 7, 33], [1, 7, 33]),                     # head size 16: half a step of the product is padding
    (5, 5, 48, 16, [2, 1, 1], [300, 17, 256]),                 # portions beside single tokens: both kernels, one call
    (8, 1, 32, 16, [64, 1], [64, 513]),                        # 8 heads on one kv head
    (6, 3, 80, 4, [3, 5], [40, 5]),                            # pages of 4
    (32, 8, 128, 16, [1, 1, 1, 1], [700, 1, 257, 16]),         # decoding only: splits and their reduction
    (32, 8, 128, 16, [130, 40], [130, 1000]),                  # several tiles per request, a long context before one
    (40, 2, 64, 16, [1, 9], [300, 64]),                        # 20 heads per kv head: more than one block of heads
    (2, 1, 256, 32, [9, 1], [70, 2000]),
    (3, 1, 112, 16, [17], [129]),
]


@pytest.mark.parametrize("shape", MFMA_SHAPES)
@pytest.mark.parametrize("window", [0, 24, 200])
def test_paged_attention_matrix_core_kernels(ops, ref, shape, window):
    nh, nkv, d, ps, seg_lens, ctx_lens = shape
    q, kp, vp, bt, seg, pos = _paged_case(torch.bfloat16, nh, nkv, d, ps, seg_lens, ctx_lens, seed=nh + d + ps, spike=True)
    scale = 1.0 / math.sqrt(d)
    a = ops.paged_attention(q, kp, vp, bt, seg, pos, nh, nkv, d, scale, window, kernel="mfma")
    b = ref.paged_attention(q, kp, vp, bt, seg, pos, nh, nkv, d, scale, window)
    c = ops.paged_attention(q, kp, vp, bt, seg, pos, nh, nkv, d, scale, window, kernel="generic")
    assert torch.allclose(a.float(), b.float(), **tol(torch.bfloat16)), (a.float() - b.float()).abs().max()
    assert torch.allclose(c.float(), b.float(), **tol(torch.bfloat16)), (c.float() - b.float()).abs().max()


@pytest.mark.parametrize("ps,first,window", [(8, 16400, 0), (16, 16380, 0), (32, 16385, 0), (8, 16400, 5000)])
def test_prefill_attention_beyond_the_block_tables_window(ops, ref, ps, first, window):
    """The LDS-staged prefill kernel keeps 2,048 entries of a request's block table in LDS at a time (64 in the form
    for tests) and moves that window on as it walks the keys: portions of a prompt that stand after so many tokens
    that the table is longer than the window (more than 2,048 pages of 8 tokens; with 64 entries, pages of 16 and 32
    too), beside a short request, and with a sliding window that starts deep inside the table. One far key per kv
    head stands out, so a page looked up in the wrong window would show."""
    nh, nkv, d = 4, 2, 32
    scale = 1.0 / math.sqrt(d)
    seg_lens, ctx_lens = [70, 33, 5], [first + 70, 100, first // 2]
    q, kp, vp, bt, seg, pos = _paged_case(torch.bfloat16, nh, nkv, d, ps, seg_lens, ctx_lens, seed=ps + first, spike=True)
    # a key far from the start stands out too: in the third window of 64 entries, and beyond 2,048 pages of 8 tokens
    far = first - 7
    kp[int(bt[0, far // ps]), :, far % ps, :] *= 5.0
    assert ps > 8 or bt.shape[1] > 2048
    want = ref.paged_attention(q, kp, vp, bt, seg, pos, nh, nkv, d, scale, window)
    for variant in (0, 2):
        ops.prefill_attention_variant = variant
        try:
            got = ops.paged_attention(q, kp, vp, bt, seg, pos, nh, nkv, d, scale, window, kernel="mfma")
        finally:
            ops.prefill_attention_variant = 0
        assert torch.allclose(got.float(), want.float(), **tol(torch.bfloat16)), \
            (variant, (got.float() - want.float()).abs().max())


@pytest.mark.parametrize("shape", MFMA_SHAPES)
@pytest.mark.parametrize("variant,splits", [(1, 1), (0, 3), (1, 64), (2, 1)])
def test_matrix_core_attention_other_ways_of_cutting_the_work(ops, ref, shape, variant, splits):
    """The forms that the planner picks only for other workloads: every wave fetching keys and values for itself
    (prefill), the keys of a single token in one part, in three, in as many as there are 128-key chunks."""
    nh, nkv, d, ps, seg_lens, ctx_lens = shape
    q, kp, vp, bt, seg, pos = _paged_case(torch.bfloat16, nh, nkv, d, ps, seg_lens, ctx_lens, seed=7 * nh + d, spike=True)
    scale = 1.0 / math.sqrt(d)
    b = ref.paged_attention(q, kp, vp, bt, seg, pos, nh, nkv, d, scale, 0)
    ops.prefill_attention_variant, ops.decode_attention_splits = variant, splits
    try:
        a = ops.paged_attention(q, kp, vp, bt, seg, pos, nh, nkv, d, scale, 0, kernel="mfma")
    finally:
        ops.prefill_attention_variant, ops.decode_attention_splits = 0, 0
    assert torch.allclose(a.float(), b.float(), **tol(torch.bfloat16)), (a.float() - b.float()).abs().max()


@pytest.mark.parametrize("d,ps", [(64, 16), (96, 8), (128, 16), (128, 32), (160, 16)])
def test_prefill_attention_every_number_of_steps(ops, ref, d, ps):
    """The LDS-staged prefill kernel walks the keys in steps of 32 through a ring of three or four stages, its
    loop unrolled by the stages, with the pages of the steps ahead looked up in a padded copy of the block table:
    prompts of 1 to 12 steps (every remainder of the ring, a last page that is full, one that holds a single
    token), alone and after a context, in head sizes that run with eight waves of 16 rows (64, 128), four of 32
    (96) and three stages (160)."""
    nh, nkv = 4, 2
    scale = 1.0 / math.sqrt(d)
    for seg_lens, ctx_lens in (([1, 31, 32, 33], [1, 31, 32, 33]), ([64, 65, 95], [64, 65, 95]),
                               ([128, 129, 97], [128, 129, 97]), ([160, 200, 256], [160, 200, 256]),
                               ([290, 383], [290, 383]), ([3, 40, 17], [99, 232, 385]), ([33], [321])):
        q, kp, vp, bt, seg, pos = _paged_case(torch.bfloat16, nh, nkv, d, ps, seg_lens, ctx_lens,
                                              seed=d + ps + sum(ctx_lens), spike=True)
        want = ref.paged_attention(q, kp, vp, bt, seg, pos, nh, nkv, d, scale, 0)
        got = ops.paged_attention(q, kp, vp, bt, seg, pos, nh, nkv, d, scale, 0, kernel="mfma")
        assert torch.allclose(got.float(), want.float(), **tol(torch.bfloat16)), \
            (seg_lens, ctx_lens, (got.float() - want.float()).abs().max())
        for window in (33, 100):
            want = ref.paged_attention(q, kp, vp, bt, seg, pos, nh, nkv, d, scale, window)
            got = ops.paged_attention(q, kp, vp, bt, seg, pos, nh, nkv, d, scale, window, kernel="mfma")
            assert torch.allclose(got.float(), want.float(), **tol(torch.bfloat16)), \
                (seg_lens, ctx_lens, window, (got.float() - want.float()).abs().max())


def test_matrix_core_attention_random_geometries(ops):
    """Sixty random geometries (heads, groups, head sizes in steps of 16, page sizes, windows, mixes of single
    tokens and portions of prompts after contexts of any length): the matrix-core kernels against the general
    kernel, which the other tests hold against the plain implementation."""
    g = torch.Generator().manual_seed(2024)

    def pick(options):
        return options[int(torch.randint(0, len(options), (1,), generator=g))]

    for case in range(60):
        nkv = pick([1, 2, 3, 8])
        nh = nkv * pick([1, 2, 4, 5])
        d = pick([16, 32, 48, 64, 80, 96, 112, 128, 160, 256])
        ps = pick([4, 8, 16, 32, 64])
        window = pick([0, 0, 7, 64, 300])
        n_seg = pick([1, 2, 3, 5])
        seg_lens, ctx_lens = [], []
        for _ in range(n_seg):
            new = pick([1, 1, 2, 17, 33, 70, 130])
            before = pick([0, 0, 1, 15, 31, 32, 100, 257, 600])
            seg_lens.append(new)
            ctx_lens.append(new + before)
        q, kp, vp, bt, seg, pos = _paged_case(torch.bfloat16, nh, nkv, d, ps, seg_lens, ctx_lens, seed=case, spike=True)
        scale = 1.0 / math.sqrt(d)
        a = ops.paged_attention(q, kp, vp, bt, seg, pos, nh, nkv, d, scale, window, kernel="mfma")
        b = ops.paged_attention(q, kp, vp, bt, seg, pos, nh, nkv, d, scale, window, kernel="generic")
        err = (a.float() - b.float()).abs().max().item()
        assert torch.allclose(a.float(), b.float(), **tol(torch.bfloat16)), \
            (case, nh, nkv, d, ps, window, seg_lens, ctx_lens, err)


@pytest.mark.parametrize("order", [1, 2])
@pytest.mark.parametrize("B,ps", [(19, 8), (7, 8), (19, 32), (7, 64)])
def test_decode_attention_in_a_given_order_of_tokens(ops, ref, order, B, ps):
    """A step of single tokens whose contexts differ, with the tokens listed longest context first and either
    arrangement of the workgroups: the same result as in the order they come in. (In such a step the kernel takes
    token i as request i without looking the request up, and below 16 tokens it does not go through the list.)"""
    from types import SimpleNamespace
    g = torch.Generator().manual_seed(21 + B)
    nh, nkv, d = 6, 3, 48
    lens = [int(x) for x in torch.randint(1, 300, (B,), generator=g)]
    per = [-(-n // ps) for n in lens]
    pages = sum(per) + 3
    kp = dev(torch.randn(pages, nkv, ps, d, generator=g).to(torch.bfloat16))
    vp = dev(torch.randn(pages, nkv, d, ps, generator=g).to(torch.bfloat16))
    perm = torch.randperm(pages, generator=g).to(torch.int32)
    bt = torch.zeros(B, max(per) + 2, dtype=torch.int32)
    at = 0
    for i, n in enumerate(per):
        bt[i, :n] = perm[at:at + n]
        at += n
    q = dev(torch.randn(B, (nh + 2 * nkv) * d, generator=g).to(torch.bfloat16))
    seg = dev(torch.arange(B, dtype=torch.int32))
    pos = dev(torch.tensor([n - 1 for n in lens], dtype=torch.int32))
    want = ref.paged_attention(q, kp, vp, dev(bt), seg, pos, nh, nkv, d, d ** -0.5)
    batch = SimpleNamespace(aux={}, host_seg_lens=[1] * B, host_seg_starts=list(range(B + 1)),
                            host_seg_first_pos=[n - 1 for n in lens], max_context=512, replayed=False, all_single=True,
                            n_tokens=B, longest_first=torch.argsort(pos, descending=True, stable=True).to(torch.int32))
    ops.decode_attention_order = order
    try:
        got = ops.paged_attention(q, kp, vp, dev(bt), seg, pos, nh, nkv, d, d ** -0.5, batch=batch, kernel="mfma")
    finally:
        ops.decode_attention_order = 0
    assert torch.allclose(got.float(), want.float(), **tol(torch.bfloat16)), (got.float() - want.float()).abs().max()
    plain = ops.paged_attention(q, kp, vp, dev(bt), seg, pos, nh, nkv, d, d ** -0.5, kernel="mfma")
    assert torch.equal(got, plain)


@pytest.mark.parametrize("nh,nkv,d,ps", [(4, 2, 16, 8), (5, 5, 48, 16), (6, 3, 80, 4), (8, 2, 128, 16), (2, 1, 256, 32), (3, 1, 112, 16),
                                         (8, 2, 128, 32), (5, 5, 48, 64), (6, 3, 80, 128), (4, 2, 64, 24)])
@pytest.mark.parametrize("window", [0, 700])
def test_decode_attention_reduction_over_many_splits(ops, ref, nh, nkv, d, ps, window):
    """More than 16 splits of a long context are added up by groups of lanes that take every G-th split (up to
    16: one loop per output element); requests of other lengths in the same call use fewer of the splits, and a
    window leaves the first ones without keys. Pages of 32 tokens and more run in the form of the kernel that deals
    a step's keys so that a lane's eight are eight in a row."""
    ctx_lens = [2500, 1, 2300, 130]
    q, kp, vp, bt, seg, pos = _paged_case(torch.bfloat16, nh, nkv, d, ps, [1, 1, 1, 1], ctx_lens, seed=nh + d, spike=True)
    scale = 1.0 / math.sqrt(d)
    b = ref.paged_attention(q, kp, vp, bt, seg, pos, nh, nkv, d, scale, window)
    ops.decode_attention_splits = 64
    try:
        a = ops.paged_attention(q, kp, vp, bt, seg, pos, nh, nkv, d, scale, window, kernel="mfma")
    finally:
        ops.decode_attention_splits = 0
    assert torch.allclose(a.float(), b.float(), **tol(torch.bfloat16)), (a.float() - b.float()).abs().max()


@pytest.mark.parametrize("nh,nkv,d,ps", [(8, 2, 128, 16), (4, 4, 64, 8), (6, 2, 80, 16)])
@pytest.mark.parametrize("trend", ["rising", "falling", "jump"])
def test_prefill_attention_moves_its_reference_when_scores_run_away(ops, ref, nh, nkv, d, ps, trend):
    """The prefill kernel takes its exponentials against a reference that it moves only when a row's scores have
    risen 2^24 above it. Keys whose scores rise steadily, fall steadily, or jump once by far more than that
    (in units of log2: hundreds) must give the plain result: every key a multiple of one direction that all
    queries share, so that the score of key j is the multiple."""
    T = 200
    g = torch.Generator().manual_seed(nh * d + len(trend))
    q, kp, vp, bt, seg, pos = _paged_case(torch.bfloat16, nh, nkv, d, ps, [T], [T], seed=5)
    u = torch.randn(d, generator=g)
    u = u / u.norm()
    scale = 1.0 / math.sqrt(d)
    # score of key j for every query = 8 * amp[j] * scale^-1 * scale = 8 amp[j] (natural log units)
    amp = {"rising": torch.linspace(-40.0, 40.0, T), "falling": torch.linspace(40.0, -40.0, T),
           "jump": torch.cat([torch.full((T // 2,), -30.0), torch.full((T - T // 2,), 30.0)])}[trend]
    qn = torch.zeros(T, nh * d + 8)
    for h in range(nh):
        qn[:, h * d:(h + 1) * d] = 8.0 * u / scale ** 0.5
    kn = kp.float().cpu()
    for j in range(T):
        page, off = int(bt[0, j // ps]), j % ps
        kn[page, :, off, :] = (amp[j] * u / scale ** 0.5) + 0.05 * torch.randn(nkv, d, generator=g)
    q, kp = dev(qn.bfloat16()), dev(kn.bfloat16())
    b = ref.paged_attention(q, kp, vp, bt, seg, pos, nh, nkv, d, scale, 0)
    a = ops.paged_attention(q, kp, vp, bt, seg, pos, nh, nkv, d, scale, 0, kernel="mfma")
    assert torch.isfinite(a.float()).all()
    assert torch.allclose(a.float(), b.float(), **tol(torch.bfloat16)), (a.float() - b.float()).abs().max()


def test_matrix_core_attention_refuses_what_it_cannot_do(ops):
    q, kp, vp, bt, seg, pos = _paged_case(torch.bfloat16, 2, 1, 24, 16, [3], [3], seed=1)
    with pytest.raises(ValueError, match="multiple of 16"):
        ops.paged_attention(q, kp, vp, bt, seg, pos, 2, 1, 24, 0.2, kernel="mfma")
    out = ops.paged_attention(q, kp, vp, bt, seg, pos, 2, 1, 24, 0.2)      # the general kernel takes it
    assert torch.isfinite(out.float()).all()


def test_decode_attention_finds_a_far_key(ops):
    """One key among thousands, in an early page, carries the answer; every split but one sees noise."""
    nh, nkv, d, ps, ctx = 8, 2, 128, 16, 5000
    g = torch.Generator().manual_seed(3)
    pages = -(-ctx // ps)
    perm = torch.randperm(pages, generator=g)
    bt = perm.to(torch.int32)[None, :]
    kp = torch.randn(pages, nkv, ps, d, generator=g) * 0.1
    vp = torch.randn(pages, nkv, d, ps, generator=g) * 0.1
    q = torch.randn(1, nh * d, generator=g)
    far = 37
    page, off = int(perm[far // ps]), far % ps
    for h in range(nkv):
        kp[page, h, off] = q[0, h * (nh // nkv) * d:h * (nh // nkv) * d + d] * 4.0     # matches the group's first head
        vp[page, h, :, off] = 5.0
    args = (dev(q.bfloat16()), dev(kp.bfloat16()), dev(vp.bfloat16()), dev(bt), dev(torch.zeros(1, dtype=torch.int32)),
            dev(torch.tensor([ctx - 1], dtype=torch.int32)), nh, nkv, d, 1.0 / math.sqrt(d))
    out = ops.paged_attention(*args, kernel="mfma").float().cpu().view(nh, d)
    for h in range(nkv):
        assert (out[h * (nh // nkv)] - 5.0).abs().max() < 0.1      # softmax is all on the far key
    with_window = ops.paged_attention(*args, 64, kernel="mfma").float().cpu().view(nh, d)
    assert with_window.abs().max() < 1.0                           # out of the window: gone


@pytest.mark.parametrize("dtype", DTYPES)
def test_paged_attention_reduces_to_library_softmax(ops, dtype):
    """One request, one head, no rotation: the kernel must equal softmax(q k^T / sqrt d) v of torch."""
    d, ps, T = 64, 16, 50
    g = torch.Generator().manual_seed(1)
    q = torch.randn(T, d, generator=g).to(dtype)
    k = torch.randn(T, d, generator=g).to(dtype)
    v = torch.randn(T, d, generator=g).to(dtype)
    pages = -(-T // ps)
    kp = torch.zeros(pages, 1, ps, d, dtype=dtype)
    kp.view(pages * ps, d)[:T] = k
    vt = torch.zeros(pages * ps, d, dtype=dtype)
    vt[:T] = v
    vp = vt.view(pages, 1, ps, d).transpose(2, 3).contiguous()
    bt = torch.arange(pages, dtype=torch.int32)[None, :]
    out = ops.paged_attention(dev(q), dev(kp), dev(vp), dev(bt), dev(torch.zeros(T, dtype=torch.int32)),
                              dev(torch.arange(T, dtype=torch.int32)), 1, 1, d, 1.0 / math.sqrt(d))
    want = torch.nn.functional.scaled_dot_product_attention(q.float()[None], k.float()[None], v.float()[None],
                                                            is_causal=True)[0]
    assert torch.allclose(out.float().cpu(), want, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["silu", "gelu"])
@pytest.mark.parametrize("N,I", [(3, 176), (17, 14336), (1, 5)])
def test_gated_act(ops, ref, dtype, kind, N, I):
    g = torch.Generator().manual_seed(I)
    gu = dev((torch.randn(N, 2 * I, generator=g) * 4).to(dtype))
    a, b = ops.gated_act(gu, kind), ref.gated_act(gu, kind)
    assert torch.allclose(a.float(), b.float(), **tol(dtype))


@pytest.mark.parametrize("M,N,K", [(1, 1000, 128), (7, 331, 80), (65, 64, 176), (130, 257, 1030), (33, 4096, 4096)])
@pytest.mark.parametrize("bias", [False, True])
def test_linear_float32_is_exact_float32(ops, M, N, K, bias):
    """The float32 product must agree with a float64 product to the rounding of a float32 sum of K terms:
    results are of size sqrt(K), each of the K additions rounds by up to 2^-24 of that, and the roundings
    add like a random walk, so the largest error among many outputs stays below 2^-24 K times a small
    factor. A reduced-precision matrix mode (10 or 7 bits of mantissa in the inputs) would miss this bound
    by a factor of 30 or more."""
    g = torch.Generator().manual_seed(M * N + K)
    x, w = torch.randn(M, K, generator=g), torch.randn(N, K, generator=g)
    b = torch.randn(N, generator=g) if bias else None
    y = ops.linear(dev(x), dev(w), dev(b) if bias else None)
    want = x.double() @ w.double().t() + (b.double() if bias else 0)
    err = (y.cpu().double() - want).abs().max().item()
    assert err < 6e-8 * K * 5, err


@pytest.mark.parametrize("M,N,K", [(1, 1000, 128), (7, 331, 80), (64, 640, 352), (65, 512, 176), (300, 1024, 512),
                                   (17, 328, 128), (33, 4096, 4096), (64, 6144, 4096), (48, 1000, 14336), (64, 4096, 1024),
                                   (65, 4096, 4096), (96, 1000, 14336), (97, 328, 128), (128, 6144, 4096), (127, 4096, 1024),
                                   (200, 1000, 1024), (129, 4096, 4096), (130, 328, 192), (192, 6144, 4096),
                                   (256, 4096, 14336), (255, 1000, 128), (300, 6144, 4096), (2048, 1000, 1024),
                                   # a K that is no multiple of 8 (even and odd): no streaming kernel takes it
                                   (1, 333, 11100), (3, 130, 331), (8, 4160, 1004), (13, 77, 2001), (16, 520, 250),
                                   (17, 130, 331), (100, 77, 1004)])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_linear_bfloat16(ops, ref, M, N, K, bias, out_dtype):
    g = torch.Generator().manual_seed(M + N + K)
    x = dev(torch.randn(M, K, generator=g).to(torch.bfloat16))
    w = dev((torch.randn(N, K, generator=g) * 0.1).to(torch.bfloat16))
    b = dev(torch.randn(N, generator=g).to(torch.bfloat16)) if bias else None
    y = ops.linear(x, w, b, out_dtype=out_dtype)
    want = ref.linear(x, w, b, out_dtype=torch.float32)
    assert y.dtype == out_dtype
    t = dict(atol=1e-4, rtol=1e-4) if out_dtype == torch.float32 else dict(atol=3e-2, rtol=1.6e-2)
    assert torch.allclose(y.float(), want, **t), (y.float() - want).abs().max()


@pytest.mark.parametrize("M", [1, 2, 8, 16, 24, 64, 100, 128, 200, 256, 300, 600, 2048])
def test_products_over_a_weight_whose_rows_lie_apart(ops, M):
    """The engine lays a weight's rows out further apart than they are long (`weight_row_pad`) and fills what is
    between with nothing: every product, for every number of rows, plain and gated, bfloat16 and float32, gives over
    such a weight the bits that it gives over the same rows lying back to back, whatever lies between them."""
    assert ops.weight_row_pad_bytes % 16 == 0
    g = torch.Generator().manual_seed(M)
    for (N, K, gated) in ((384, 512, False), (4096, 1024, False), (1024, 3072, False), (704, 256, True),
                          (2048, 1024, True)):
        for dtype in (torch.bfloat16, torch.float32):
            if dtype == torch.float32 and (M > 64 or N * K > 1 << 20):
                continue
            pad = ops.weight_row_pad(K, dtype)
            assert pad > 0 and pad * torch.empty((), dtype=dtype).element_size() == ops.weight_row_pad_bytes
            x = dev(torch.randn(M, K, generator=g).to(dtype))
            w = dev((torch.randn(N, K, generator=g) * K ** -0.5).to(dtype))
            buf = torch.full((N, K + pad), float("nan"), dtype=dtype, device=w.device)
            apart = buf[:, :K]
            apart.copy_(w)
            f = (lambda t: ops.linear_gated(x, t, None, "silu")) if gated else (lambda t: ops.linear(x, t))
            a, b = f(w), f(apart)
            assert torch.equal(a, b) and not torch.isnan(b.float()).any(), (M, N, K, gated, dtype)
            if not gated:
                a32, b32 = ops.linear(x, w, out_dtype=torch.float32), ops.linear(x, apart, out_dtype=torch.float32)
                assert torch.equal(a32, b32), (M, N, K, dtype)


@pytest.mark.parametrize("M,I,K", [(1, 176, 64), (8, 14336, 4096), (16, 208, 80), (13, 1000, 328), (40, 352, 128),
                                   (64, 14336, 4096), (20, 1000, 1024), (65, 14336, 4096), (100, 1000, 1024),
                                   (129, 352, 128), (200, 14336, 4096), (256, 1000, 192), (300, 1000, 1024),
                                   # outputs that are 4 modulo 8, 2 modulo 4 and odd, at every kernel's numbers of rows
                                   (8, 1004, 192), (40, 1004, 192), (100, 1004, 192), (200, 11100, 4160), (100, 250, 64),
                                   (40, 331, 128), (130, 331, 128)])
@pytest.mark.parametrize("kind", ["silu", "gelu"])
@pytest.mark.parametrize("bias", [False, True])
def test_linear_gated(ops, ref, M, I, K, kind, bias):
    """The gated feed-forward's first half: with few rows the activation is the product's epilogue. It must
    give the bits of the product followed by the activation kernel, and both the plain formula."""
    g = torch.Generator().manual_seed(M * I + K)
    x = dev((torch.randn(M, K, generator=g)).bfloat16())
    w = dev((torch.randn(2 * I, K, generator=g) * K ** -0.5).bfloat16())
    b = dev(torch.randn(2 * I, generator=g).bfloat16()) if bias else None
    fused = ops.linear_gated(x, w, b, kind)
    two = ops.gated_act(ops.linear(x, w, b), kind)
    assert fused.shape == (M, I) and fused.dtype == torch.bfloat16
    if M <= 16 or K <= 512:
        if 2 < M <= 16:
            # the default tilings split K over 8 waves (gated) and 16 (plain): equal up to a rounding of the
            # sums; with the plain product's 8-wave tiling the order of summation is the same and so are the bits
            assert (fused.float() - two.float()).abs().max().item() <= 2e-2 * max(1.0, two.float().abs().max().item())
            ops.skinny_variant = 2
            try:
                fused, two = ops.linear_gated(x, w, b, kind), ops.gated_act(ops.linear(x, w, b), kind)
            finally:
                ops.skinny_variant = 0
        assert torch.equal(fused, two)           # the same order of summation in both
    else:
        # more than 16 rows and a long K: the two may split K differently, which moves a sum by a rounding
        assert (fused.float() - two.float()).abs().max().item() <= 2e-2 * max(1.0, two.float().abs().max().item())
    want = ref.linear_gated(x.float(), w.float(), None if b is None else b.float(), kind)
    assert (fused.float() - want).abs().max().item() <= 2e-2 * max(1.0, want.abs().max().item())
    f32 = ops.linear_gated(x.float(), w.float(), None if b is None else b.float(), kind)      # float32: no fusion, no rounding
    assert f32.dtype == torch.float32 and torch.allclose(f32, want, atol=1e-4, rtol=1e-4)


@pytest.mark.parametrize("M,H,nh,nkv,d,ps", [(1, 128, 8, 1, 32, 16), (8, 4096, 32, 8, 128, 16), (16, 80, 3, 3, 64, 8),
                                             (5, 256, 4, 2, 96, 4), (2, 4096, 32, 8, 128, 16), (1, 5000, 5, 5, 64, 8),
                                             (2, 640, 6, 2, 32, 4)])
@pytest.mark.parametrize("bias", [False, True])
def test_qkv_rope_cache_fused_equals_the_three_steps(ops, ref, M, H, nh, nkv, d, ps, bias):
    """With few rows the rotation and the cache write are the epilogue of the QKV product; the result must be
    the bits of product, rotation kernel and cache write one after the other, and the plain formulas."""
    g = torch.Generator().manual_seed(M * H + d)
    N = (nh + 2 * nkv) * d
    x = dev(torch.randn(M, H, generator=g).bfloat16())
    w = dev((torch.randn(N, H, generator=g) * H ** -0.5).bfloat16())
    b = dev(torch.randn(N, generator=g).bfloat16()) if bias else None
    max_pos, pages = 50, 7
    pos = dev(torch.randint(0, max_pos, (M,), generator=g, dtype=torch.int32))
    ang = torch.arange(max_pos, dtype=torch.float32)[:, None] * torch.rand(d // 2, generator=g)[None, :]
    table = dev(torch.cat([ang.cos(), ang.sin()], dim=1).contiguous())
    slots = torch.randperm(pages * ps, generator=g)[:M].to(torch.int32)
    if M > 2:
        slots[2] = -1
    slots = dev(slots)
    k1, v1 = dev(torch.zeros(pages, nkv, ps, d).bfloat16()), dev(torch.zeros(pages, nkv, d, ps).bfloat16())
    k2, v2, k3, v3 = k1.clone(), v1.clone(), k1.clone(), v1.clone()
    fused = ops.qkv_rope_cache(x, w, b, nh, nkv, d, pos, table, d, True, slots, k1, v1)
    # (two rows: the fused form streams W without the matrix cores, the plain product does so row by row)
    steps = ops.linear(x, w, b) if M != 2 else torch.cat([ops.linear(x[m:m + 1], w, b) for m in range(M)])
    ops.rope_cache_write(steps, nh, nkv, d, pos, table, d, True, slots, k2, v2)
    assert torch.equal(fused, steps) and torch.equal(k1, k2) and torch.equal(v1, v2)
    plain = ref.qkv_rope_cache(x, w, b, nh, nkv, d, pos, table, d, True, slots, k3, v3)
    scale = max(1.0, plain.float().abs().max().item())
    assert (fused.float() - plain.float()).abs().max().item() <= 2e-2 * scale
    assert (k1.float() - k3.float()).abs().max().item() <= 2e-2 * scale and (v1.float() - v3.float()).abs().max().item() <= 2e-2 * scale
    # what the fused kernel does not take falls back to the three steps: GPT-J pairing, partial rotation
    k4, v4, k5, v5 = k3.clone().zero_(), v3.clone().zero_(), k3.clone().zero_(), v3.clone().zero_()
    a = ops.qkv_rope_cache(x, w, b, nh, nkv, d, pos, table[:, :d // 2].contiguous(), d // 2, False, slots, k4, v4)
    c = ref.qkv_rope_cache(x, w, b, nh, nkv, d, pos, table[:, :d // 2].contiguous(), d // 2, False, slots, k5, v5)
    assert (a.float() - c.float()).abs().max().item() <= 2e-2 * scale and (k4.float() - k5.float()).abs().max().item() <= 2e-2 * scale


@pytest.mark.parametrize("M", [17, 24, 32, 33, 48, 49, 64])
@pytest.mark.parametrize("H,nh,nkv,d,ps", [(4096, 32, 8, 128, 16), (1024, 6, 3, 64, 8), (320, 5, 5, 32, 4)])
@pytest.mark.parametrize("bias", [False, True])
def test_qkv_rope_cache_in_the_few_rows_kernel_beyond_16_rows(ops, ref, M, H, nh, nkv, d, ps, bias):
    """The QKV product with rotation and cache write as epilogue takes up to 64 rows in the few-rows kernel (two to
    four tiles of rows; the switch point ``qkv_fused_max_rows`` says up to where it is used): against the plain
    formulas, and within a rounding of the 17-and-more-rows product followed by the rotary kernel, which adds up K in
    another order."""
    g = torch.Generator().manual_seed(M + H + d)
    N = (nh + 2 * nkv) * d
    x = dev(torch.randn(M, H, generator=g).bfloat16())
    w = dev((torch.randn(N, H, generator=g) * H ** -0.5).bfloat16())
    b = dev(torch.randn(N, generator=g).bfloat16()) if bias else None
    max_pos, pages = 70, -(-M // ps) + 3
    pos = dev(torch.randint(0, max_pos, (M,), generator=g, dtype=torch.int32))
    ang = torch.arange(max_pos, dtype=torch.float32)[:, None] * torch.rand(d // 2, generator=g)[None, :]
    table = dev(torch.cat([ang.cos(), ang.sin()], dim=1).contiguous())
    slots = torch.randperm(pages * ps, generator=g)[:M].to(torch.int32)
    slots[M - 1] = -1
    slots = dev(slots)
    k1, v1 = dev(torch.zeros(pages, nkv, ps, d).bfloat16()), dev(torch.zeros(pages, nkv, d, ps).bfloat16())
    k2, v2, k3, v3 = k1.clone(), v1.clone(), k1.clone(), v1.clone()
    before = ops.qkv_fused_max_rows
    try:
        ops.qkv_fused_max_rows = 64
        fused = ops.qkv_rope_cache(x, w, b, nh, nkv, d, pos, table, d, True, slots, k1, v1)
        ops.qkv_fused_max_rows = 0
        apart = ops.qkv_rope_cache(x, w, b, nh, nkv, d, pos, table, d, True, slots, k2, v2)
    finally:
        ops.qkv_fused_max_rows = before
    plain = ref.qkv_rope_cache(x, w, b, nh, nkv, d, pos, table, d, True, slots, k3, v3)
    scale = max(1.0, plain.float().abs().max().item())
    for got, want in ((fused, plain), (k1, k3), (v1, v3), (fused, apart), (k1, k2), (v1, v2)):
        assert (got.float() - want.float()).abs().max().item() <= 2e-2 * scale
    assert not torch.equal(k1, torch.zeros_like(k1))


@pytest.mark.parametrize("M,N,K", [(17, 256, 1024), (40, 4096, 4096), (64, 80, 1280), (33, 1000, 2048), (65, 256, 1024),
                                   (100, 4096, 4096), (128, 80, 1280)])
@pytest.mark.parametrize("bias", [False, True])
def test_unfinished_product_is_finished_by_the_norm(ops, ref, M, N, K, bias):
    """A product of 17 to 64 rows whose K is split may stay as partial sums; the norm that takes it as its
    branch adds them up. The bits are those of product, then addition and norm, and the plain formulas hold."""
    from lmsf_amd.ops.handles import PendingProduct
    g = torch.Generator().manual_seed(M + N + K)
    x = dev(torch.randn(M, K, generator=g).bfloat16())
    w = dev((torch.randn(N, K, generator=g) * K ** -0.5).bfloat16())
    b = dev(torch.randn(N, generator=g).bfloat16()) if bias else None
    p = ops.linear(x, w, b, pending_ok=True)
    assert isinstance(p, PendingProduct) and p.shape == (M, N) and p.partials.shape[0] >= 2
    y = ops.linear(x, w, b)
    assert torch.equal(ops.materialize(p), y) and ops.materialize(y) is y
    nw = dev(torch.randn(N, generator=g).bfloat16())
    res0 = dev(torch.randn(M, N, generator=g))
    for out_dtype, weight in ((torch.bfloat16, nw), (torch.float32, nw.float())):
        r1, r2 = res0.clone(), res0.clone()
        a = ops.add_rms_norm(p, r1, weight, 1e-5, out_dtype, weight_offset=0.25)
        c = ops.add_rms_norm(y, r2, weight, 1e-5, out_dtype, weight_offset=0.25)
        assert torch.equal(a, c) and torch.equal(r1, r2) and not torch.equal(r1, res0)
        want = ref.add_rms_norm(y, res0.clone(), weight, 1e-5, torch.float32, weight_offset=0.25)
        assert (a.float() - want).abs().max().item() <= 2e-2 * max(1.0, want.abs().max().item())
    rows = dev(torch.tensor([M - 1, 0, 5], dtype=torch.int32))
    r1 = res0.clone()
    a = ops.add_rms_norm(p, r1, nw, 1e-5, torch.bfloat16, rows=rows)
    c = ops.add_rms_norm(y, res0.clone(), nw, 1e-5, torch.bfloat16, rows=rows)
    assert torch.equal(a, c) and torch.equal(r1, res0)
    # without a residual: the norm of the product alone
    assert torch.equal(ops.add_rms_norm(p, None, nw, 1e-5, torch.bfloat16), ops.add_rms_norm(y, None, nw, 1e-5, torch.bfloat16))


@pytest.mark.parametrize("M,H,nh,nkv,d,ps,rot,neox", [(17, 1024, 8, 2, 64, 16, 64, True), (64, 4096, 32, 8, 128, 16, 128, True),
                                                      (40, 1024, 6, 3, 48, 8, 24, False), (33, 1280, 5, 5, 80, 4, 80, False),
                                                      (100, 4096, 32, 8, 128, 16, 128, True), (128, 1024, 6, 3, 48, 8, 24, False)])
@pytest.mark.parametrize("bias", [False, True])
def test_qkv_rope_cache_from_partial_sums(ops, ref, M, H, nh, nkv, d, ps, rot, neox, bias):
    """With 17 to 64 rows the QKV product splits K, and the rotation kernel adds up the partial sums before it
    rotates and stores: the bits are those of product, rotation and cache write one after the other."""
    g = torch.Generator().manual_seed(M * H + d)
    N = (nh + 2 * nkv) * d
    x = dev(torch.randn(M, H, generator=g).bfloat16())
    w = dev((torch.randn(N, H, generator=g) * H ** -0.5).bfloat16())
    b = dev(torch.randn(N, generator=g).bfloat16()) if bias else None
    assert ops.lib.lmsf_gemm_mid_splits(M, N, H, 0) >= 2
    max_pos, pages = 50, -(-M // ps) + 3
    pos = dev(torch.randint(0, max_pos, (M,), generator=g, dtype=torch.int32))
    ang = torch.arange(max_pos, dtype=torch.float32)[:, None] * torch.rand(rot // 2, generator=g)[None, :]
    table = dev(torch.cat([ang.cos(), ang.sin()], dim=1).contiguous())
    slots = torch.randperm(pages * ps, generator=g)[:M].to(torch.int32)
    slots[2] = -1
    slots = dev(slots)
    k1, v1 = dev(torch.zeros(pages, nkv, ps, d).bfloat16()), dev(torch.zeros(pages, nkv, d, ps).bfloat16())
    k2, v2, k3, v3 = k1.clone(), v1.clone(), k1.clone(), v1.clone()
    fused = ops.qkv_rope_cache(x, w, b, nh, nkv, d, pos, table, rot, neox, slots, k1, v1)
    steps = ops.linear(x, w, b)
    ops.rope_cache_write(steps, nh, nkv, d, pos, table, rot, neox, slots, k2, v2)
    assert torch.equal(fused, steps) and torch.equal(k1, k2) and torch.equal(v1, v2)
    plain = ref.qkv_rope_cache(x, w, b, nh, nkv, d, pos, table, rot, neox, slots, k3, v3)
    scale = max(1.0, plain.float().abs().max().item())
    assert (fused.float() - plain.float()).abs().max().item() <= 2e-2 * scale
    assert (k1.float() - k3.float()).abs().max().item() <= 2e-2 * scale and (v1.float() - v3.float()).abs().max().item() <= 2e-2 * scale
    # no rotation and no cache: the product alone
    assert torch.equal(ops.qkv_rope_cache(x, w, b, nh, nkv, d, pos, None, 0, True, None, None, None), ops.linear(x, w, b))
    # no rotation, cache write only
    k4, v4, k5, v5 = k1.clone().zero_(), v1.clone().zero_(), k1.clone().zero_(), v1.clone().zero_()
    a = ops.qkv_rope_cache(x, w, b, nh, nkv, d, pos, None, 0, True, slots, k4, v4)
    c = ops.linear(x, w, b)
    ops.rope_cache_write(c, nh, nkv, d, pos, None, 0, True, slots, k5, v5)
    assert torch.equal(a, c) and torch.equal(k4, k5) and torch.equal(v4, v5)


@pytest.mark.parametrize("M", [1, 2])
@pytest.mark.parametrize("N,K", [(1000, 128), (331, 80), (4096, 4096), (520, 14336), (77, 5000), (64, 4608)])
@pytest.mark.parametrize("bias", [False, True])
def test_products_of_one_or_two_rows(ops, ref, M, N, K, bias):
    """One or two rows stream W without the matrix cores (a wave per row of W, x in LDS, K in pieces of 4,096
    with the last piece partial): plain with both output types, gated, and the fused QKV form, against the
    plain formulas and against the few-rows kernel, which adds up K in another order."""
    g = torch.Generator().manual_seed(N + K + M)
    x = dev(torch.randn(M, K, generator=g).bfloat16())
    w = dev((torch.randn(2 * N, K, generator=g) * K ** -0.5).bfloat16())
    b = dev(torch.randn(2 * N, generator=g).bfloat16()) if bias else None
    assert ops.gemv_max_rows >= 2
    try:
        for out_dtype in (torch.bfloat16, torch.float32):
            b1 = b[:N] if bias else None
            want = ref.linear(x, w[:N], b1, torch.float32)
            ops.gemv_max_rows = 2
            a = ops.linear(x, w[:N], b1, out_dtype=out_dtype)
            ops.gemv_max_rows = 0
            c = ops.linear(x, w[:N], b1, out_dtype=out_dtype)
            t = (2e-2 if out_dtype == torch.bfloat16 else 2e-3) * max(1.0, want.abs().max().item())
            assert a.dtype == out_dtype and (a.float() - want).abs().max().item() <= t
            assert (a.float() - c.float()).abs().max().item() <= t
        for kind in ("silu", "gelu"):
            want = ref.linear_gated(x, w, b, kind).float()
            ops.gemv_max_rows = 2
            a = ops.linear_gated(x, w, b, kind)
            # the bits of product (one row: the same kernel without epilogue), rounding, activation kernel
            steps = ops.gated_act(torch.cat([ops.linear(x[m:m + 1], w, b) for m in range(M)]), kind)
            assert torch.equal(a, steps)
            assert (a.float() - want).abs().max().item() <= 2e-2 * max(1.0, want.abs().max().item())
    finally:
        ops.gemv_max_rows = 2


@pytest.mark.parametrize("M", [3, 8, 16])
@pytest.mark.parametrize("H,I", [(1024, 14300), (4096, 14336), (256, 16384), (512, 28600), (8192, 14336)])
@pytest.mark.parametrize("bias", [False, True])
def test_gated_product_after_a_norm_in_either_kernel(ops, ref, M, H, I, bias):
    """The gated product that applies the norm's row factor itself runs in the 17-and-more-rows kernel where that
    kernel's workgroups fit on the chip at once, else in the few-rows kernel: the two agree with each other and with
    the plain formula, with outputs that are no multiple of 64 and with a bias; so does the form with 128 outputs a
    workgroup, which takes over where workgroups of 64 outputs would be more than the chip holds at once."""
    from lmsf_amd.ops.handles import ScaledRows
    g = torch.Generator().manual_seed(M * H + I)
    x = dev(torch.randn(M, H, generator=g).bfloat16())
    w = dev((torch.randn(H, H, generator=g) * H ** -0.5).bfloat16())
    nw = dev(torch.randn(H, generator=g).bfloat16())
    res = dev(torch.randn(M, H, generator=g) * 3.0)
    p = ops.linear(x, w, None, pending_ok=True)
    h = ops.add_rms_norm(p, res.clone(), nw, 1e-5, torch.bfloat16, defer_ok=True)
    assert isinstance(h, ScaledRows) and h.rows_per_tile == 16
    wg = dev((torch.randn(2 * I, H, generator=g) * H ** -0.5).bfloat16())
    bg = dev(torch.randn(2 * I, generator=g).bfloat16()) if bias else None
    # the form with 128 outputs a workgroup is chosen beyond 8 rows only; asked for directly it takes any number
    assert ops.lib.lmsf_gemm_mid_scaled_fits(M, I, H, h.tiles) == (1 if I <= 16384 or M > 8 else 0)
    assert ops.lib.lmsf_gemm_mid_scaled_fits(16, I, H, h.tiles) == 1
    want_h = ref.add_rms_norm(ops.linear(x, w), res.clone(), nw, 1e-5, torch.bfloat16)
    for kind in ("silu", "gelu"):
        if ops.lib.lmsf_gemm_mid_scaled_fits(M, I, H, h.tiles):
            here = ops.linear_gated(h, wg, bg, kind)
        else:
            from lmsf_amd.ops.hip_ops import _ptr
            here = torch.empty((M, I), dtype=torch.bfloat16, device=h.xw.device)
            ops._check(ops.lib.lmsf_gemm_mid_scaled(
                _ptr(h.xw), h.xw.stride(0), _ptr(wg), wg.stride(0), _ptr(bg), _ptr(here), here.stride(0), M, I, H,
                {"silu": 1, "gelu": 2}[kind], _ptr(h.sumsq), h.tiles, h.eps, ops._stream()))
        before = ops.mid_scaled_rows
        ops.mid_scaled_rows = 0
        try:
            there = ops.linear_gated(h, wg, bg, kind)
        finally:
            ops.mid_scaled_rows = before
        want = ref.linear_gated(want_h, wg, bg, kind).float()
        t = 2e-2 * max(1.0, want.abs().max().item())
        assert here.shape == (M, I) and (here.float() - want).abs().max().item() <= t
        assert (here.float() - there.float()).abs().max().item() <= t and not torch.isnan(here.float()).any()
    # too many workgroups for the chip, too few to keep most of it busy, or sums of squares that a thread cannot hold:
    # the few-rows kernel
    assert ops.lib.lmsf_gemm_mid_scaled_fits(8, 11008, H, h.tiles) == 0 and ops.lib.lmsf_gemm_mid_scaled_fits(16, 11008, H, h.tiles) == 1
    assert ops.lib.lmsf_gemm_mid_scaled_fits(16, 2048, H, h.tiles) == 0
    assert ops.lib.lmsf_gemm_mid_scaled_fits(M, 64 * 257, H, h.tiles) == 0
    assert ops.lib.lmsf_gemm_mid_scaled_fits(M, 128 * 257, H, h.tiles) == 0
    assert ops.lib.lmsf_gemm_mid_scaled_fits(M, I, 16384, 1024) == 0 and ops.lib.lmsf_gemm_mid_scaled_fits(17, I, H, h.tiles) == 0


@pytest.mark.parametrize("M,stream_rows", [(1, 1), (2, 2), (2, 1), (8, 1), (16, 1)])
@pytest.mark.parametrize("H,K,nh,nkv,d,I", [(4096, 4096, 32, 8, 128, 1024), (1000, 14336, 5, 5, 64, 331), (80, 128, 3, 1, 32, 77),
                                            (8200, 256, 2, 2, 64, 96)])
@pytest.mark.parametrize("bias", [False, True])
def test_norm_done_by_the_products_around_it(ops, ref, M, stream_rows, H, K, nh, nkv, d, I, bias):
    """With up to 16 rows the product before a norm adds its rounded result into the float32 stream and leaves
    bf16(stream * w) and sums of squares over parts of the columns (16 columns each from the few-rows kernel,
    a workgroup's share from the kernel for one or two rows); the product after it multiplies its rows by
    rsqrt(sum / H + eps). The stream gets the bits of product, then addition; the products agree with the norm
    kernel's path up to where the rounding to bfloat16 falls."""
    before = ops.fuse_stream_rows
    ops.fuse_stream_rows = stream_rows      # rows up to which the kernel for one or two rows is taken
    try:
        _norm_done_by_the_products(ops, ref, M, H, K, nh, nkv, d, I, bias, gemv=M <= stream_rows)
    finally:
        ops.fuse_stream_rows = before


def _norm_done_by_the_products(ops, ref, M, H, K, nh, nkv, d, I, bias, gemv):
    from lmsf_amd.ops.handles import DeferredLinear, ScaledRows
    g = torch.Generator().manual_seed(M + H + K)
    x = dev(torch.randn(M, K, generator=g).bfloat16())
    w = dev((torch.randn(H, K, generator=g) * K ** -0.5).bfloat16())
    b = dev(torch.randn(H, generator=g).bfloat16()) if bias else None
    nw = dev(torch.randn(H, generator=g).bfloat16())
    res0 = dev(torch.randn(M, H, generator=g) * 3.0)
    p = ops.linear(x, w, b, pending_ok=True)
    assert isinstance(p, DeferredLinear) and p.shape == (M, H)
    # (the product as the same kernel stores it: row by row for the kernel of one or two rows)
    y = torch.cat([ops.linear(x[m:m + 1], w, b) for m in range(M)]) if gemv else ops.linear(x, w, b)
    assert gemv or torch.equal(ops.materialize(p), y)
    r1, r2 = res0.clone(), res0.clone()
    h = ops.add_rms_norm(p, r1, nw, 1e-5, torch.bfloat16, weight_offset=0.25, defer_ok=True)
    c = ops.add_rms_norm(y, r2, nw, 1e-5, torch.bfloat16, weight_offset=0.25)
    assert torch.equal(r1, r2) and not torch.equal(r1, res0)
    assert isinstance(h, ScaledRows) and h.shape == (M, H) and h.stream is r1
    assert (h.rows_per_tile, h.tiles) == ((M, ops.lib.lmsf_gemv_partials(H)) if gemv else (16, -(-H // 16)))
    # what it holds: stream * w rounded, and sums of squares that add up to the rows' own
    assert torch.equal(h.xw, (r1 * (nw.float() + 0.25)).bfloat16())
    sums = h.sumsq.view(h.tiles, h.rows_per_tile).sum(0)
    want_sums = (r1.double() ** 2).sum(1)
    assert torch.allclose(sums[:M].double(), want_sums, rtol=1e-5) and (M == h.rows_per_tile or float(sums[M:].abs().max()) == 0.0)
    assert torch.equal(ops.materialize(h), c)
    want_h = ref.add_rms_norm(y, res0.clone(), nw, 1e-5, torch.bfloat16, weight_offset=0.25)
    wg = dev((torch.randn(2 * I, H, generator=g) * H ** -0.5).bfloat16())
    bg = dev(torch.randn(2 * I, generator=g).bfloat16()) if bias else None
    for kind in ("silu", "gelu"):
        a = ops.linear_gated(h, wg, bg, kind)
        want = ref.linear_gated(want_h, wg, bg, kind).float()
        t = 2e-2 * max(1.0, want.abs().max().item())
        assert a.shape == (M, I) and (a.float() - want).abs().max().item() <= t
        assert (a.float() - ops.linear_gated(c, wg, bg, kind).float()).abs().max().item() <= t
    N = (nh + 2 * nkv) * d
    wq = dev((torch.randn(N, H, generator=g) * H ** -0.5).bfloat16())
    bq = dev(torch.randn(N, generator=g).bfloat16()) if bias else None
    max_pos, pages, ps = 50, 5, 8
    pos = dev(torch.randint(0, max_pos, (M,), generator=g, dtype=torch.int32))
    ang = torch.arange(max_pos, dtype=torch.float32)[:, None] * torch.rand(d // 2, generator=g)[None, :]
    table = dev(torch.cat([ang.cos(), ang.sin()], dim=1).contiguous())
    slots = torch.randperm(pages * ps, generator=g)[:M].to(torch.int32)
    if M > 2:
        slots[1] = -1
    slots = dev(slots)
    k1, v1 = dev(torch.zeros(pages, nkv, ps, d).bfloat16()), dev(torch.zeros(pages, nkv, d, ps).bfloat16())
    k2, v2 = k1.clone(), v1.clone()
    a = ops.qkv_rope_cache(h, wq, bq, nh, nkv, d, pos, table, d, True, slots, k1, v1)
    want = ref.qkv_rope_cache(want_h, wq, bq, nh, nkv, d, pos, table, d, True, slots, k2, v2)
    t = 2e-2 * max(1.0, want.float().abs().max().item())
    assert (a.float() - want.float()).abs().max().item() <= t
    assert (k1.float() - k2.float()).abs().max().item() <= t and (v1.float() - v2.float()).abs().max().item() <= t
    assert k1.float().abs().sum().item() > 0
    # what the fused forms do not take sees the norm kernel's output: GPT-J pairing
    k3, v3, k4, v4 = k1.clone().zero_(), v1.clone().zero_(), k1.clone().zero_(), v1.clone().zero_()
    a = ops.qkv_rope_cache(h, wq, bq, nh, nkv, d, pos, table[:, :d // 2].contiguous(), d // 2, False, slots, k3, v3)
    e = ops.qkv_rope_cache(c, wq, bq, nh, nkv, d, pos, table[:, :d // 2].contiguous(), d // 2, False, slots, k4, v4)
    assert torch.equal(a, e) and torch.equal(k3, k4)
    # the caller that does not take it, selected rows, a float32 norm weight: the norm kernel
    r3 = res0.clone()
    assert torch.equal(ops.add_rms_norm(p, r3, nw, 1e-5, torch.bfloat16, weight_offset=0.25), c) and torch.equal(r3, r1)
    rows = dev(torch.tensor([M - 1], dtype=torch.int32))
    r4 = res0.clone()
    a = ops.add_rms_norm(p, r4, nw, 1e-5, torch.bfloat16, rows=rows, weight_offset=0.25, defer_ok=True)
    assert torch.is_tensor(a) and torch.equal(r4, res0)
    # (selected rows finish the product with the few-rows kernel, which for two rows adds up K in another order)
    assert torch.equal(a, c[M - 1:]) or (gemv and M == 2 and (a.float() - c[M - 1:].float()).abs().max().item() <= 2e-2 * 10)
    r5 = res0.clone()
    assert torch.is_tensor(ops.add_rms_norm(p, r5, nw.float(), 1e-5, torch.bfloat16, weight_offset=0.25, defer_ok=True))


def test_split_heuristic_counts_the_gated_forms_extra_kernel(ops):
    """Splitting K fills the chip when there are few rows of W, at the price of partial sums and, for the gated
    form, a kernel that adds them up: at a feed-forward's sizes (224 workgroups without a split) that price is
    never worth it, at an o projection's (64 workgroups) it always is."""
    for M in (17, 18, 24, 32, 64):
        assert ops.lib.lmsf_gemm_mid_splits(M, 14336, 4096, 1) == 1
        assert ops.lib.lmsf_gemm_mid_splits(M, 4096, 4096, 0) >= 4
        assert ops.lib.lmsf_gemm_mid_splits(M, 4096, 14336, 0) >= 4


@pytest.mark.parametrize("M,N,K", [(129, 4096, 4096), (192, 4096, 14336), (256, 6144, 4096), (150, 328, 192),
                                   (256, 136, 64), (65, 1000, 1024), (300, 128, 448), (512, 1024, 3072), (1000, 256, 768)])
def test_linear_many_rows_every_tiling_and_split(ops, ref, M, N, K):
    """The many-rows product (csrc/gemm_large.hip) with each of its tilings, in one piece and with K split into
    parts whose float32 partial sums are added up by the reduction kernel or stay for the norm that follows: all
    against the float32 product, and a split product against the unsplit one of the same tiling."""
    from lmsf_amd.ops.handles import PendingProduct
    g = torch.Generator().manual_seed(M + N + K)
    x = dev(torch.randn(M, K, generator=g).to(torch.bfloat16))
    w = dev((torch.randn(N, K, generator=g) * K ** -0.5).to(torch.bfloat16))
    b = dev(torch.randn(N, generator=g).to(torch.bfloat16))
    want = ref.linear(x, w, b, out_dtype=torch.float32)
    scale = want.abs().max().item()
    for tiling in (0, 1, 2, 3, 4, 5):            # (3 to 5: the tiles of 0 to 2 with two groups of four waves)
        whole = ops._linear_large(x, w, b, 0, plan=tiling * 16 + 1)
        assert (whole.float() - want).abs().max().item() <= 1e-2 * scale, tiling
        for parts in (2, 3, 8):
            if parts > K // 64:
                continue
            got = ops._linear_large(x, w, b, 0, plan=tiling * 16 + parts)
            assert (got.float() - whole.float()).abs().max().item() <= 1e-2 * scale, (tiling, parts)
            pending = ops._linear_large(x, w, b, 0, pending_ok=True, plan=tiling * 16 + parts)
            assert isinstance(pending, PendingProduct) and pending.partials.shape == (parts, M, N)
            assert torch.equal(ops.materialize(pending), got)
    plan = ops.lib.lmsf_gemm_large_plan(M, N, K, 0)
    assert 0 <= plan // 16 <= 5 and 1 <= plan % 16 <= 8
    # what the engine calls: the same numbers through linear, and as the branch of a norm
    y = ops.linear(x, w, b)
    assert (y.float() - want).abs().max().item() <= 1e-2 * scale
    if M > ops.mid_max_rows:
        res = dev(torch.randn(M, N, generator=g))
        nw = dev(torch.randn(N, generator=g).to(torch.bfloat16))
        p = ops.linear(x, w, b, pending_ok=True)
        r1, r2 = res.clone(), res.clone()
        a = ops.add_rms_norm(p, r1, nw, 1e-5, torch.bfloat16)
        c = ops.add_rms_norm(y, r2, nw, 1e-5, torch.bfloat16)
        assert torch.equal(a, c) and torch.equal(r1, r2)


@pytest.mark.parametrize("bias", [False, True])
def test_library_products_race_for_a_shape(ops, bias):
    """The BLAS library's candidates for one shape race on three copies of the weight and the winner is kept for that
    shape (one plan more, none for its neighbours). Whatever algorithm runs, the product is the product: the raced
    shape and others of the same weight against float32."""
    g = torch.Generator().manual_seed(9)
    N, K = 1536, 1024
    pad = ops.weight_row_pad(K, torch.bfloat16)
    weights = []
    for _ in range(3):
        buf = dev(torch.zeros(N, K + pad).bfloat16())
        buf[:, :K].copy_(dev((torch.randn(N, K, generator=g) * K ** -0.5).bfloat16()))
        weights.append(buf[:, :K])
    b = dev(torch.randn(N, generator=g).bfloat16()) if bias else None
    x = dev(torch.randn(2048, K, generator=g).bfloat16())
    plans = ops.lib.lmsf_blas_plans()
    first, best = ops.tune_products(x[:1024], weights, b, candidates=8, reps=3)
    assert 0 < best <= first < 1e5
    assert ops.lib.lmsf_blas_plans() == plans + 1
    for M in (1024, 1000, 513, 2048, 300):
        got = ops.linear(x[:M], weights[1], b)
        want = x[:M].float() @ weights[1].float().t() + (b.float() if bias else 0.0)
        assert (got.float() - want).abs().max().item() <= 2e-2 * max(1.0, want.abs().max().item()), M
    # a race needs operands of one shape
    with pytest.raises(ValueError, match="one shape"):
        ops.tune_products(x[:512], [weights[0], weights[1][:8]], b)


def test_linear_mixed_storage(ops, ref):
    """A weight stored in 32 bits stays so and still multiplies bfloat16 activations."""
    g = torch.Generator().manual_seed(5)
    x = dev(torch.randn(5, 96, generator=g).to(torch.bfloat16))
    w = dev(torch.randn(40, 96, generator=g))
    y = ops.linear(x, w)
    assert y.dtype == torch.bfloat16
    assert torch.allclose(y.float(), ref.linear(x, w, None, torch.float32), atol=5e-2, rtol=1e-2)


@pytest.mark.parametrize("V", [256, 1000, 128256])
def test_sample_greedy_and_seeded(ops, ref, V):
    g = torch.Generator().manual_seed(V)
    R = 6
    logits = torch.randn(R, V, generator=g) * 3
    logits[0, 5] = logits[0, 77] = 50.0                 # a tie: the lowest index wins
    lg = dev(logits)
    assert ops.sample(lg).tolist() == torch.argmax(logits, dim=-1).tolist() and ops.sample(lg)[0].item() == 5
    temp = dev(torch.tensor([0.0, 0.7, 1.0, 1.3, 0.7, 0.7]))
    top_k = dev(torch.tensor([-1, -1, 5, 50, -1, 3], dtype=torch.int32))
    top_p = dev(torch.tensor([1.0, 1.0, 1.0, 0.9, 0.5, 0.8]))
    min_p = dev(torch.tensor([0.0, 0.0, 0.0, 0.0, 0.0, 0.05]))
    seeds = dev(torch.tensor([1, 2, 3, 4, 5, 2 ** 40 + 17], dtype=torch.int64))
    for draw in range(3):
        draws = dev(torch.full((R,), draw, dtype=torch.int32))
        a = ops.sample(lg, temp, top_k, top_p, min_p, seeds, draws)
        b = ref.sample(lg, temp, top_k, top_p, min_p, seeds, draws)
        assert a.tolist() == b.tolist(), (draw, a.tolist(), b.tolist())


@pytest.mark.parametrize("V", [1000, 128256])
def test_sample_top_p_alone_on_peaked_and_flat_rows(ops, ref, V):
    """Top-p without a top-k: peaked rows (few entries can be kept: they are gathered once) and flat rows (most
    of the row can be kept: the passes over the whole row) give the plain sampler's tokens."""
    g = torch.Generator().manual_seed(V + 1)
    scales = [0.5, 2.0, 6.0, 9.0, 14.0, 9.0, 9.0, 0.0]
    R = len(scales)
    logits = torch.randn(R, V, generator=g) * torch.tensor(scales)[:, None]
    logits[6, 3] = logits[6].max() + 30.0                  # one entry holds all the mass
    lg = dev(logits)
    temp = dev(torch.tensor([1.0, 0.8, 1.0, 1.2, 1.0, 0.6, 1.0, 1.0]))
    top_p = dev(torch.tensor([0.9, 0.95, 0.9, 0.5, 0.999, 0.05, 0.9, 0.7]))
    seeds = dev(torch.arange(100, 100 + R, dtype=torch.int64))
    for draw in range(4):
        draws = dev(torch.full((R,), draw, dtype=torch.int32))
        a = ops.sample(lg, temp, None, top_p, None, seeds, draws)
        b = ref.sample(lg, temp, None, top_p, None, seeds, draws)
        assert a.tolist() == b.tolist(), (draw, a.tolist(), b.tolist())
        assert a[6].item() == 3


@pytest.mark.parametrize("extreme", [False, True])
def test_sample_rows_and_settings_drawn_at_random(ops, ref, extreme):
    """Rows and settings drawn at random (vocabularies of 50 to 128,256, flat to peaked rows, many equal values,
    one entry far above the rest; with ``extreme`` also masked entries, huge values and temperatures of 2e-5
    to 50) give the plain sampler's tokens. A sweep like this is what found a noise value of +inf and zeros
    of two signs with two keys."""
    import random
    for it in range(40):
        rng = random.Random(it + (1000 if extreme else 0))
        V = rng.choice([50, 777, 1000, 5000, 32000, 128256])
        R = rng.choice([1, 3, 8])
        g = torch.Generator().manual_seed(it)
        scales = torch.tensor([rng.choice([0.0, 0.1, 1.0, 3.0, 8.0, 15.0]) for _ in range(R)])
        logits = torch.randn(R, V, generator=g) * scales[:, None]
        if rng.random() < 0.3:
            logits = (logits * 4).round() / 4
        if rng.random() < 0.3:
            logits[0, rng.randrange(V)] += 40.0
        if extreme:
            if rng.random() < 0.5:
                logits[torch.rand(R, V, generator=g) < 0.3] = float("-inf")
                logits[:, rng.randrange(V)] = 1.0
            if rng.random() < 0.3:
                logits = logits * 1e4
        temps = [0.0, 0.3, 0.7, 1.0, 1.5] + ([1e-4, 2e-5, 50.0] if extreme else [])
        args = [dev(torch.tensor([rng.choice(temps) for _ in range(R)])),
                dev(torch.tensor([rng.choice([-1, 1, 2, 5, 50, 1000, 1024, 1025, 5000]) for _ in range(R)], dtype=torch.int32)),
                dev(torch.tensor([rng.choice([1.0, 0.99, 0.9, 0.5, 0.1, 0.01]) for _ in range(R)])),
                dev(torch.tensor([rng.choice([0.0, 0.0, 0.01, 0.3]) for _ in range(R)])),
                dev(torch.tensor([rng.randrange(2 ** 48) for _ in range(R)], dtype=torch.int64))]
        lg = dev(logits)
        for draw in range(2):
            draws = dev(torch.full((R,), draw, dtype=torch.int32))
            a, b = ops.sample(lg, *args, draws).tolist(), ref.sample(lg, *args, draws).tolist()
            assert a == b, (it, draw, V, a, b, [t.tolist() for t in args[:4]])


def test_sample_noise_is_finite(ops):
    """The draw adds -log(-log(u)) to every entry; a u that rounds to 1 makes that +inf and its entry the
    winner whatever its probability. One entry holds all the mass but 1e-8 here: over 2,000 draws of 128,256
    entries each (where a u of 24 bits plus a half rounds to 1 fifteen times) it is drawn every time."""
    V, R = 128256, 500
    logits = torch.full((R, V), -30.0)
    logits[:, 77] = 0.0
    lg = dev(logits)
    temp = dev(torch.ones(R))
    seeds = dev(torch.arange(1000, 1000 + R, dtype=torch.int64))
    for draw in range(4):
        draws = dev(torch.full((R,), draw, dtype=torch.int32))
        for cuts in (None, dev(torch.full((R,), 0.999))):          # the draw over the whole row, and the kernel with cuts
            out = ops.sample(lg, temp, None, cuts, None, seeds, draws)
            assert (out == 77).all(), (draw, cuts is not None, out[out != 77].tolist())


@pytest.mark.parametrize("V", [50, 5000, 128256])
def test_sample_takes_zeros_of_either_sign_as_equal(ops, ref, V):
    """A row whose largest values are zeros of both signs (they compare equal): no cut separates them."""
    g = torch.Generator().manual_seed(V)
    R = 6
    logits = torch.randn(R, V, generator=g) * 0.0                # +0 and -0 at random
    logits[3:] -= torch.rand(3, V, generator=g).round() * 5.0     # about half of the entries far below the zeros
    assert (logits == 0).any() and torch.signbit(logits[0]).any() and not torch.signbit(logits[0]).all()
    lg = dev(logits)
    temp = dev(torch.tensor([0.7, 1.0, 0.3, 0.7, 1.0, 1.5]))
    top_k = dev(torch.tensor([1, 2, -1, 5, 1000, -1], dtype=torch.int32))
    top_p = dev(torch.tensor([1.0, 0.9, 0.1, 0.5, 0.01, 0.9]))
    min_p = dev(torch.tensor([0.0, 0.01, 0.0, 0.3, 0.0, 0.0]))
    seeds = dev(torch.arange(40, 40 + R, dtype=torch.int64))
    seen = set()
    for draw in range(6):
        draws = dev(torch.full((R,), draw, dtype=torch.int32))
        a = ops.sample(lg, temp, top_k, top_p, min_p, seeds, draws)
        b = ref.sample(lg, temp, top_k, top_p, min_p, seeds, draws)
        assert a.tolist() == b.tolist(), (draw, a.tolist(), b.tolist())
        assert all(logits[r, t] == 0 for r, t in enumerate(a.tolist()))
        seen.add(bool(torch.signbit(logits[0, a[0]])))
    assert seen == {True, False} or V == 50    # with top_k = 1 both kinds of zero are drawn


@pytest.mark.parametrize("V", [1000, 16384, 128256])
def test_greedy_takes_the_first_of_equal_maxima(ops, V):
    g = torch.Generator().manual_seed(V)
    logits = torch.randn(5, V, generator=g)
    logits[0, [V - 1, V // 2, 7]] = 9.0          # equal maxima far apart (different workgroups of a large vocabulary)
    logits[1, V - 1] = 9.0                        # the last entry
    logits[2, 0] = 9.0
    logits[3] = -1.0                              # all equal
    logits[4, V // 2 + 1] = float("inf")
    out = ops.sample(dev(logits)).cpu().tolist()
    assert out == [7, V - 1, 0, 0, V // 2 + 1]


def test_sample_does_not_depend_on_batch(ops):
    g = torch.Generator().manual_seed(9)
    logits = dev(torch.randn(4, 777, generator=g))
    temp = dev(torch.full((4,), 0.9))
    seeds = dev(torch.tensor([11, 12, 13, 14], dtype=torch.int64))
    draws = dev(torch.tensor([0, 5, 2, 9], dtype=torch.int32))
    whole = ops.sample(logits, temp, None, None, None, seeds, draws).tolist()
    for r in range(4):
        one = ops.sample(logits[r:r + 1], temp[r:r + 1], None, None, None, seeds[r:r + 1], draws[r:r + 1]).tolist()
        assert one == [whole[r]]


def test_sample_frequencies_follow_softmax(ops):
    """Over many draws the tokens come with the probabilities softmax(logits / T) gives (chi-square)."""
    V, n = 12, 4000
    g = torch.Generator().manual_seed(3)
    row = torch.randn(V, generator=g)
    T = 0.8
    p = torch.softmax(row / T, dim=-1)
    lg = dev(row[None, :].repeat(n, 1).contiguous())
    out = ops.sample(lg, dev(torch.full((n,), T)), None, None, None,
                     dev(torch.full((n,), 123, dtype=torch.int64)), dev(torch.arange(n, dtype=torch.int32)))
    counts = torch.bincount(out.cpu().long(), minlength=V).float()
    chi2 = (((counts - n * p) ** 2) / (n * p)).sum().item()
    assert chi2 < 40.0, chi2           # 11 degrees of freedom: P(chi2 > 40) < 4e-5


def test_apply_penalties(ops, ref):
    g = torch.Generator().manual_seed(4)
    R, V = 3, 500
    logits = torch.randn(R, V, generator=g)
    rows = [([1, 2, 3, 3], [3, 4, 4, 4]), ([7], []), ([], [9, 9, 499])]
    tokens, offsets, plens = [], [0], []
    for pr, out in rows:
        tokens += pr + out
        offsets.append(len(tokens))
        plens.append(len(pr))
    args = [dev(torch.tensor(tokens, dtype=torch.int32)), dev(torch.tensor(offsets, dtype=torch.int32)),
            dev(torch.tensor(plens, dtype=torch.int32)), dev(torch.tensor([0.2, 0.0, 1.0])),
            dev(torch.tensor([0.1, 0.0, 0.5])), dev(torch.tensor([1.3, 1.0, 0.8]))]
    a, b = dev(logits.clone()), dev(logits.clone())
    ops.apply_penalties(a, *args)
    ref.apply_penalties(b, *args)
    assert torch.allclose(a, b, atol=1e-6)
    assert not torch.equal(a, dev(logits))


def test_measured_rates_are_plausible(ops):
    """The yardstick kernels of bench.py run (a buffer whose size is no multiple of the grid: the last workgroup
    takes the rest) and report rates of the order of this hardware's."""
    rates = ops.measure(nbytes=(1 << 28) + 4096 * 7 + 16, reps=1)
    assert 500 < rates["read_GBps"] < 20000 and 500 < rates["copy_GBps"] < 20000
    assert 100 < rates["mfma_bf16_TFLOPs"] < 5000
