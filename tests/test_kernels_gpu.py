"""Each HIP kernel alone against its plain reference (tests/kernel_refs.py), at
sizes other than the engine's tiny models: widths that are no power of two,
group sizes 1..5, page sizes 1..32, head sizes 16..256, both dtypes."""

from __future__ import annotations

import math

import pytest
import torch

import kernel_refs as refs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from forge_engine_amd.kernels import ops as real_ops
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return real_ops


def tol(dtype):
    return dict(atol=2e-2, rtol=2e-2) if dtype == torch.bfloat16 else dict(atol=1e-5, rtol=1e-5)


def rand(gen, *shape, dtype=torch.float32, scale=1.0):
    return (torch.randn(*shape, generator=gen) * scale).to(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden", [40, 200, 2560])
def test_embed_rows(ops, dtype, hidden):
    g = torch.Generator().manual_seed(0)
    table = rand(g, 77, hidden, dtype=dtype)
    ids = torch.tensor([0, 76, 5, 5, 31], dtype=torch.int32)
    want = refs.embed_rows(ids, table, torch.empty(5, hidden))
    got = ops.embed_rows(ids.to(DEV), table.to(DEV), torch.empty(5, hidden, device=DEV))
    torch.testing.assert_close(got.cpu(), want, atol=0, rtol=0)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("delta_dtype", [None, torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden", [24, 200, 2560, 5000, 5120, 8192])
@pytest.mark.parametrize("n", [7, 23, 600])     # up to 512 rows of a wide stream take a kernel with more threads a row
def test_add_rmsnorm(ops, out_dtype, delta_dtype, hidden, n):
    g = torch.Generator().manual_seed(1)
    h = rand(g, n, hidden, scale=3.0)
    delta = None if delta_dtype is None else rand(g, n, hidden, dtype=delta_dtype)
    w = 1.0 + rand(g, hidden, scale=0.1)
    h_ref = h.clone()
    want = refs.add_rmsnorm(h_ref, delta, w, 1e-5, torch.empty(n, hidden, dtype=out_dtype))
    h_dev = h.to(DEV)
    got = ops.add_rmsnorm(h_dev, None if delta is None else delta.to(DEV), w.to(DEV), 1e-5,
                          torch.empty(n, hidden, dtype=out_dtype, device=DEV))
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(out_dtype))
    torch.testing.assert_close(h_dev.cpu(), h_ref, atol=1e-6, rtol=1e-6)   # the sum went back into the stream


def test_add_rmsnorm_reference_vectors(ops):
    # the vectors of the reference's own tests (tests/test_qwen3.py:34-44, tests/test_kernels.py:20-36)
    h = torch.tensor([[1.0, -2.0, 3.0, -4.0]])
    u = torch.tensor([[0.5, 1.0, -1.5, 2.0]])
    w = torch.tensor([1.0, 2.0, 3.0, 4.0])
    got = ops.add_rmsnorm(h.to(DEV), None, w.to(DEV), 1e-6, torch.empty(1, 4, device=DEV)).cpu()
    torch.testing.assert_close(got, h * torch.rsqrt(h.square().mean(-1, keepdim=True) + 1e-6) * w)
    h_dev = h.to(DEV)
    got = ops.add_rmsnorm(h_dev, u.to(DEV), w.to(DEV), 1e-6, torch.empty(1, 4, device=DEV)).cpu()
    s = h + u
    torch.testing.assert_close(h_dev.cpu(), s)
    torch.testing.assert_close(got, s * torch.rsqrt(s.square().mean(-1, keepdim=True) + 1e-6) * w)


def test_add_rmsnorm_row_list(ops):
    g = torch.Generator().manual_seed(2)
    h = rand(g, 9, 96)
    w = rand(g, 96)
    rows = torch.tensor([8, 0, 3, 3], dtype=torch.int32)
    want = refs.add_rmsnorm(h.clone(), None, w, 1e-6, torch.empty(4, 96), rows=rows, store_sum=False)
    got = ops.add_rmsnorm(h.to(DEV), None, w.to(DEV), 1e-6, torch.empty(4, 96, device=DEV),
                          rows=rows.to(DEV), store_sum=False)
    torch.testing.assert_close(got.cpu(), want, atol=1e-5, rtol=1e-5)
    # with an update that has not been added yet (whole, or in parts): the rows of the sum, and the
    # stream is left as it is
    for hidden, parts in ((96, 1), (2560, 1), (2560, 3), (200, 9)):
        h = rand(g, 9, hidden)
        w = rand(g, hidden)
        delta = rand(g, parts, 9, hidden) if parts > 1 else rand(g, 9, hidden)
        want = refs.add_rmsnorm(h.clone(), delta, w, 1e-6, torch.empty(4, hidden), rows=rows, store_sum=False)
        h_dev = h.to(DEV)
        got = ops.add_rmsnorm(h_dev, delta.to(DEV), w.to(DEV), 1e-6, torch.empty(4, hidden, device=DEV),
                              rows=rows.to(DEV), store_sum=False)
        torch.testing.assert_close(got.cpu(), want, atol=1e-5, rtol=1e-5)
        assert torch.equal(h_dev.cpu(), h)


def test_stream_read_touches_nothing(ops):
    data = torch.arange(4096, dtype=torch.float32, device=DEV)
    sink = torch.full((1,), 7.0, device=DEV)
    ops.stream_read(data, sink)
    torch.cuda.synchronize()
    assert sink.item() == 7.0 and torch.equal(data.cpu(), torch.arange(4096, dtype=torch.float32))
    with pytest.raises(ops.KernelError):
        ops.stream_read(data[:3], sink)              # not a multiple of 16 bytes


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_add_rows_and_swiglu(ops, dtype):
    g = torch.Generator().manual_seed(3)
    h = rand(g, 5, 136)
    d = rand(g, 5, 136, dtype=dtype)
    got = ops.add_rows(h.to(DEV), d.to(DEV)).cpu()
    torch.testing.assert_close(got, h + d.float())
    gu = rand(g, 6, 2 * 328, dtype=dtype, scale=2.0)
    want = refs.swiglu(gu, torch.empty(6, 328, dtype=dtype))
    got = ops.swiglu(gu.to(DEV), torch.empty(6, 328, dtype=dtype, device=DEV)).cpu()
    torch.testing.assert_close(got.float(), want.float(), **tol(dtype))
    # the library expression of the reference's own test (tests/test_cute_swiglu.py:18-27)
    torch.testing.assert_close(got.float(), (torch.nn.functional.silu(gu[:, :328].float()) * gu[:, 328:].float()), **tol(dtype))
    for inter in (100, 8, 9728):     # widths that are and are not a multiple of the 8-element pieces
        gu = rand(g, 37, 2 * inter, dtype=dtype, scale=2.0)
        want = refs.swiglu(gu, torch.empty(37, inter, dtype=dtype))
        got = ops.swiglu(gu.to(DEV), torch.empty(37, inter, dtype=dtype, device=DEV)).cpu()
        torch.testing.assert_close(got.float(), want.float(), **tol(dtype))


@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (3, 70, 50), (65, 129, 96), (130, 64, 2560), (17, 1003, 200), (5, 33, 7),
                                   # up to 16 rows with K a multiple of four: the weight-streaming variant
                                   (1, 9003, 2560), (3, 70, 52), (4, 2560, 4096), (8, 2560, 9728), (7, 1003, 200), (16, 330, 1028),
                                   (13, 6, 4), (9, 5, 1024),
                                   # up to 8 rows and K from 1,024: the rows of A stay in registers (K in one, two or three passes)
                                   (8, 1003, 2560), (5, 7, 1024), (8, 2561, 3072), (2, 600, 4096), (8, 300, 6148), (6, 131, 12292), (1, 70, 1500),
                                   # 9 to 64 rows and K from 1,024: the same kernel, eight rows a launch; more rows: tiles
                                   (9, 300, 2560), (40, 301, 2560), (64, 129, 1024), (17, 2561, 4096), (33, 70, 6148), (65, 70, 1024)])
def test_gemm_f32(ops, m, n, k):
    g = torch.Generator().manual_seed(4)
    a, b, bias = rand(g, m, k), rand(g, n, k), rand(g, n)
    want = refs.gemm_nt_f32(a, b, bias)
    got = ops.gemm_nt_f32(a.to(DEV), b.to(DEV), bias.to(DEV)).cpu()
    torch.testing.assert_close(got, want, atol=1e-4 * math.sqrt(k), rtol=1e-5)
    # a row's result does not depend on the rows beside it
    alone = ops.gemm_nt_f32(a[:1].to(DEV).contiguous(), b.to(DEV), bias.to(DEV)).cpu()
    def variant(rows):       # A in registers (eight rows a launch), the weight streamed past up to 16 rows, or tiles
        return "resident" if rows <= 64 and k >= 1024 and k % 4 == 0 else "rows" if rows <= 16 and k % 4 == 0 else "tiles"
    if variant(m) == variant(1):
        assert torch.equal(alone[0], got[0])        # the same variant, whose order of sums depends on K alone
    else:                                           # another order of the same sums
        torch.testing.assert_close(alone[0], got[0], atol=1e-5 * math.sqrt(k), rtol=1e-5)
    for rows in (2, 5, 9, 16, 40):                  # the variants for few rows give the same bits within their kind
        if rows < m and variant(m) != "tiles" and variant(rows) == variant(m):
            part = ops.gemm_nt_f32(a[:rows].to(DEV).contiguous(), b.to(DEV), bias.to(DEV)).cpu()
            assert torch.equal(part, got[:rows])


def test_gemm_f32_is_true_float32(ops):
    # operands whose product needs more than bfloat16's or tf32's mantissa
    a = torch.tensor([[1.0 + 2**-20, 1.0]])
    b = torch.tensor([[1.0, -1.0]])
    got = ops.gemm_nt_f32(a.to(DEV), b.to(DEV)).cpu()
    assert got.item() == pytest.approx(2**-20, rel=1e-6)


def _qk_case(g, dtype, tokens, q_heads, kv_heads, head_dim, block_size, num_blocks):
    width = (q_heads + 2 * kv_heads) * head_dim
    qkv = rand(g, tokens, width, dtype=dtype)
    qw, kw = 1.0 + rand(g, head_dim, scale=0.1), 1.0 + rand(g, head_dim, scale=0.1)
    # two sequences: tokens [0, split) belong to sequence 1 at positions 5.., the rest to sequence 0 from 0
    split = tokens // 2
    positions = torch.tensor(list(range(5, 5 + split)) + list(range(tokens - split)), dtype=torch.int32)
    token_seq = torch.tensor([1] * split + [0] * (tokens - split), dtype=torch.int32)
    need = (max(int(positions.max()) + 1, 1) + block_size - 1) // block_size
    perm = torch.randperm(num_blocks, generator=g)[: 2 * need].to(torch.int32)
    table = perm.view(2, need).contiguous()
    return qkv, qw, kw, positions, token_seq, table


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("q_heads,kv_heads,head_dim,block_size,rotary_dim", [
    (4, 2, 16, 4, 16), (6, 2, 32, 8, 32), (5, 1, 128, 16, 128), (3, 3, 64, 1, 32), (8, 2, 256, 32, 256),
    (2, 1, 48, 5, 0), (4, 2, 64, 8, 64), (32, 8, 128, 16, 128),
    (64, 16, 128, 16, 128), (20, 4, 256, 32, 256),       # more heads than a block of the vector kernel takes: two blocks a token
])
@pytest.mark.parametrize("tokens", [11, 300])       # few tokens: four heads a block; many: a block per token
def test_qk_norm_rope_write(ops, dtype, q_heads, kv_heads, head_dim, block_size, rotary_dim, tokens):
    g = torch.Generator().manual_seed(5)
    num_blocks = 2 * ((tokens + 5) // block_size + 2)
    qkv, qw, kw, positions, token_seq, table = _qk_case(g, dtype, tokens, q_heads, kv_heads, head_dim, block_size, num_blocks)
    inv_freq = None
    if rotary_dim:
        inv_freq = 1.0 / (10000.0 ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
    shape = (num_blocks, kv_heads, block_size, head_dim)
    vshape = (num_blocks, kv_heads, head_dim, block_size)      # values are stored transposed
    kp_ref, vp_ref = torch.zeros(shape, dtype=dtype), torch.zeros(vshape, dtype=dtype)
    qkv_ref = qkv.clone()
    refs.qk_norm_rope_write(qkv_ref, qw, kw, inv_freq, positions, token_seq, table, kp_ref, vp_ref,
                            q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim, rotary_dim=rotary_dim, eps=1e-6)
    qkv_dev = qkv.to(DEV)
    kp, vp = torch.zeros(shape, dtype=dtype, device=DEV), torch.zeros(vshape, dtype=dtype, device=DEV)
    ops.qk_norm_rope_write(qkv_dev, qw.to(DEV), kw.to(DEV), None if inv_freq is None else inv_freq.to(DEV),
                           positions.to(DEV), token_seq.to(DEV), table.to(DEV), kp, vp, q_heads=q_heads,
                           kv_heads=kv_heads, head_dim=head_dim, rotary_dim=rotary_dim, eps=1e-6)
    qs = q_heads * head_dim
    torch.testing.assert_close(qkv_dev.cpu()[:, :qs].float(), qkv_ref[:, :qs].float(), **tol(dtype))
    torch.testing.assert_close(kp.cpu().float(), kp_ref.float(), **tol(dtype))
    torch.testing.assert_close(vp.cpu().float(), vp_ref.float(), atol=0, rtol=0)
    assert torch.equal(qkv_dev.cpu()[:, qs:], qkv[:, qs:])   # the k and v parts of the buffer stay


def test_rotation_sign_and_pairing_on_device(ops):
    # unit vector in dim 0 at position 1, D = 4, theta 10000 -> (cos 1, 0, sin 1, 0)
    qkv = torch.zeros(1, 12)
    qkv[0, 0] = 1.0          # q
    qkv[0, 5] = 1.0          # k, dim 1
    inv_freq = torch.tensor([1.0, 0.01])
    kp, vp = torch.zeros(2, 1, 2, 4, device=DEV), torch.zeros(2, 1, 4, 2, device=DEV)
    dev = qkv.to(DEV)
    ops.qk_norm_rope_write(dev, None, None, inv_freq.to(DEV), torch.tensor([1], dtype=torch.int32, device=DEV),
                           torch.tensor([0], dtype=torch.int32, device=DEV),
                           torch.tensor([[1]], dtype=torch.int32, device=DEV), kp, vp, q_heads=1, kv_heads=1,
                           head_dim=4, rotary_dim=4, eps=1.0)
    torch.testing.assert_close(dev.cpu()[0, :4], torch.tensor([math.cos(1.0), 0.0, math.sin(1.0), 0.0]))
    torch.testing.assert_close(kp.cpu()[1, 0, 1], torch.tensor([0.0, math.cos(0.01), 0.0, math.sin(0.01)]))


def _attention_case(g, dtype, seqs, q_heads, kv_heads, head_dim, block_size, extra_width=0):
    """seqs: list of (ctx_before, q_len).  Builds pages with shuffled page ids."""
    total_q = sum(q for _, q in seqs)
    blocks_needed = [(b + q + block_size - 1) // block_size for b, q in seqs]
    num_blocks = sum(blocks_needed) + 3
    perm = torch.randperm(num_blocks, generator=g).tolist()
    width = max(blocks_needed)
    table = torch.full((len(seqs), width), -1, dtype=torch.int32)
    at = 0
    for s, n in enumerate(blocks_needed):
        table[s, :n] = torch.tensor(perm[at:at + n], dtype=torch.int32)
        at += n
    shape = (num_blocks, kv_heads, block_size, head_dim)
    kp, vp = rand(g, *shape, dtype=dtype), rand(g, num_blocks, kv_heads, head_dim, block_size, dtype=dtype)   # values transposed
    q = rand(g, total_q, q_heads * head_dim + extra_width, dtype=dtype)
    cu = torch.tensor([0] + list(torch.tensor([q for _, q in seqs]).cumsum(0)), dtype=torch.int32)
    ctx = torch.tensor([b + q for b, q in seqs], dtype=torch.int32)
    return q, kp, vp, cu, ctx, table


def _run_attention(ops, q, kp, vp, cu, ctx, table, *, q_heads, kv_heads, head_dim, window=None, scale=None):
    scale = head_dim ** -0.5 if scale is None else scale
    num_seqs = ctx.numel()
    max_q = int((cu[1:] - cu[:-1]).max())
    kw = dict(num_seqs=num_seqs, max_q_len=max_q, q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim,
              scale=scale, window=window)
    want = refs.paged_attention(q, kp, vp, torch.empty(q.shape[0], q_heads * head_dim, dtype=q.dtype), cu, ctx, table, **kw)
    got = ops.paged_attention(q.to(DEV), kp.to(DEV), vp.to(DEV),
                              torch.empty(q.shape[0], q_heads * head_dim, dtype=q.dtype, device=DEV),
                              cu.to(DEV), ctx.to(DEV), table.to(DEV), **kw)
    return got.cpu().float(), want.float()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("q_heads,kv_heads,head_dim,block_size", [
    (4, 2, 16, 4), (6, 2, 32, 8), (10, 2, 128, 16), (5, 5, 64, 1), (3, 1, 256, 32), (7, 1, 48, 3), (16, 1, 16, 64),
])
def test_paged_attention_mixed_batch(ops, dtype, q_heads, kv_heads, head_dim, block_size):
    g = torch.Generator().manual_seed(6)
    seqs = [(0, 37), (70, 1), (13, 9), (0, 1), (130, 2), (63, 1)]
    case = _attention_case(g, dtype, seqs, q_heads, kv_heads, head_dim, block_size, extra_width=2 * kv_heads * head_dim)
    got, want = _run_attention(ops, *case, q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim)
    torch.testing.assert_close(got, want, **tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("q_heads,kv_heads,head_dim,block_size", [
    (2, 1, 4, 2), (3, 3, 6, 4), (4, 2, 10, 16), (6, 2, 24, 8), (5, 1, 72, 16), (2, 2, 200, 16), (9, 3, 2, 5),
])
def test_paged_attention_any_even_head_size(ops, dtype, q_heads, kv_heads, head_dim, block_size):
    """Head sizes that are no multiple of 16 (the reference's own tiny test model has heads of 4)
    and rows that are not 16-byte aligned: the general kernel takes them one element at a time."""
    g = torch.Generator().manual_seed(11)
    seqs = [(0, 19), (33, 1), (7, 5), (0, 1), (64, 2)]
    case = _attention_case(g, dtype, seqs, q_heads, kv_heads, head_dim, block_size, extra_width=2 * kv_heads * head_dim)
    got, want = _run_attention(ops, *case, q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim)
    torch.testing.assert_close(got, want, **tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("q_heads,kv_heads,head_dim,block_size", [(32, 8, 128, 16), (4, 2, 16, 4), (6, 2, 48, 8), (3, 1, 256, 32)])
def test_paged_attention_general_kernel_cuts_long_contexts_into_runs(ops, dtype, q_heads, kv_heads, head_dim, block_size, monkeypatch):
    """Few sequences with long contexts: the general kernel cuts every row's keys into runs walked
    by blocks of their own and merges them; any number of runs gives the plain result (runs that
    hold no tile included), with a window too."""
    g = torch.Generator().manual_seed(12)
    seqs = [(700, 1), (0, 1), (1023, 1), (130, 3)]
    q, kp, vp, cu, ctx, table = _attention_case(g, dtype, seqs, q_heads, kv_heads, head_dim, block_size,
                                                extra_width=2 * kv_heads * head_dim)
    if dtype == torch.bfloat16:
        q = q[:, :q_heads * head_dim + 1][:, :q_heads * head_dim]      # rows 2 bytes off 16-byte alignment: not a case for the fast kernels
    for window in (None, 100):
        kw = dict(num_seqs=len(seqs), max_q_len=3, q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim,
                  scale=head_dim ** -0.5, window=window)
        want = refs.paged_attention(q, kp, vp, torch.empty(q.shape[0], q_heads * head_dim, dtype=q.dtype), cu, ctx, table, **kw).float()
        seen = []
        for runs in (1, 2, 5, 64):
            monkeypatch.setattr(ops, "generic_splits", lambda *a, runs=runs: seen.append(runs) or runs)
            got = ops.paged_attention(q.to(DEV), kp.to(DEV), vp.to(DEV),
                                      torch.full((q.shape[0], q_heads * head_dim), float("nan"), dtype=q.dtype, device=DEV),
                                      cu.to(DEV), ctx.to(DEV), table.to(DEV), num_decode=None, max_ctx=1024, **kw).cpu().float()
            torch.testing.assert_close(got, want, **tol(dtype))
        assert seen == [1, 2, 5, 64] or dtype == torch.bfloat16
    monkeypatch.undo()
    assert ops.generic_splits(8, 8, 4, 1, 128, 1040) == 8 and ops.generic_splits(64, 8, 4, 1, 128, 1040) == 1
    assert ops.generic_splits(1, 1, 1, 1, 16, 100) == 1 and ops.generic_splits(1, 8, 4, 1, 128, None) == 1


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("q_heads,kv_heads,head_dim,block_size", [
    (32, 8, 128, 16), (4, 2, 16, 4), (6, 2, 36, 12), (5, 1, 100, 20), (12, 1, 64, 8), (3, 3, 4, 4), (16, 2, 200, 16), (9, 1, 256, 32),
])
def test_vector_alu_decode_attention(ops, dtype, q_heads, kv_heads, head_dim, block_size, monkeypatch):
    """Single tokens whose shapes the matrix-core decode kernel does not take (float32; bfloat16 with
    other head sizes, pages or groups) go to the kernel that keeps keys and values out of LDS: every
    head size that is a multiple of four (16, 32 or 64 lanes a key), up to 4 or 8 heads a block and
    more in row tiles, pages of any multiple of four slots, any number of key runs (runs without
    keys included), a window, contexts at the edges of pages and tiles, and NaN in every slot that
    no live key owns."""
    g = torch.Generator().manual_seed(14)
    seqs = [(700, 1), (0, 1), (1023, 1), (63, 1), (64, 1), (130, 3), (15, 1)]
    q, kp, vp, cu, ctx, table = _attention_case(g, dtype, seqs, q_heads, kv_heads, head_dim, block_size,
                                                extra_width=2 * kv_heads * head_dim)
    if dtype == torch.bfloat16 and head_dim in (64, 128, 256) and q_heads // kv_heads <= 8 and block_size >= 16:
        block_size_ok = False     # the matrix-core kernel would take these: nothing to test here
    else:
        block_size_ok = True
    taken = []
    real_call = ops._call
    monkeypatch.setattr(ops, "_call", lambda lib, name, *a: taken.append(name) or real_call(lib, name, *a))
    for window in (None, 100):
        kw = dict(num_seqs=len(seqs), max_q_len=3, q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim,
                  scale=head_dim ** -0.5, window=window)
        want = refs.paged_attention(q, kp, vp, torch.empty(q.shape[0], q_heads * head_dim, dtype=q.dtype), cu, ctx, table, **kw).float()
        first = [0 if window is None else max(0, before - window + 1) for before, _ in seqs]
        kp_bad, vp_bad, table_bad = kp.clone(), vp.clone(), table.clone()
        _poison_unowned_slots(kp_bad, vp_bad, table, first, [b + n for b, n in seqs], block_size)
        for s, low in enumerate(first):
            table_bad[s, :low // block_size] = -1
        for runs in (1, 2, 5, 64):
            monkeypatch.setattr(ops, "rows_splits", lambda *a, runs=runs: runs)
            got = ops.paged_attention(q.to(DEV), kp_bad.to(DEV), vp_bad.to(DEV),
                                      torch.full((q.shape[0], q_heads * head_dim), float("nan"), dtype=q.dtype, device=DEV),
                                      cu.to(DEV), ctx.to(DEV), table_bad.to(DEV), num_decode=None, max_ctx=1024, **kw).cpu().float()
            assert torch.isfinite(got).all()
            torch.testing.assert_close(got, want, **tol(dtype))
    assert ("fe_paged_attention_rows" in taken) == block_size_ok
    monkeypatch.undo()
    assert ops.rows_splits(8, 8, 4, 128, 1040) == 16 and ops.rows_splits(64, 8, 4, 128, 1040) == 2
    assert ops.rows_splits(1, 1, 1, 16, 100) == 1 and ops.rows_splits(1, 8, 4, 128, None) == 1


@pytest.mark.parametrize("window", [1, 5, 16, 40])
def test_paged_attention_window(ops, window):
    g = torch.Generator().manual_seed(7)
    seqs = [(0, 50), (45, 1), (30, 7)]
    case = _attention_case(g, torch.float32, seqs, 4, 2, 32, 8)
    got, want = _run_attention(ops, *case, q_heads=4, kv_heads=2, head_dim=32, window=window)
    torch.testing.assert_close(got, want, atol=1e-5, rtol=1e-5)


def test_paged_attention_is_library_attention(ops):
    # whole prompt, nothing cached: the library's causal attention after group expansion
    # (the reference pins its own kernels the same way, tests/test_kernels.py:91-105)
    g = torch.Generator().manual_seed(8)
    q, kp, vp, cu, ctx, table = _attention_case(g, torch.float32, [(0, 21)], 6, 2, 32, 8)
    got, _ = _run_attention(ops, q, kp, vp, cu, ctx, table, q_heads=6, kv_heads=2, head_dim=32)
    keys = refs.gather_pages(kp, table[0], 21, 8)
    values = refs.gather_pages(vp.transpose(2, 3), table[0], 21, 8)
    lib = torch.nn.functional.scaled_dot_product_attention(
        q.view(21, 6, 32).transpose(0, 1).unsqueeze(0), keys.repeat_interleave(3, 0).unsqueeze(0),
        values.repeat_interleave(3, 0).unsqueeze(0), is_causal=True)[0]
    torch.testing.assert_close(got, lib.transpose(0, 1).reshape(21, 192), atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_paged_attention_far_key_stands_out(ops, dtype):
    # one key among hundreds, early in the sequence and in the middle of a page,
    # gets a score far above the rest: the output must be its value row
    g = torch.Generator().manual_seed(9)
    head_dim, block_size, ctx_len = 64, 16, 700
    q, kp, vp, cu, ctx, table = _attention_case(g, dtype, [(ctx_len - 1, 1)], 2, 1, head_dim, block_size)
    q = q * 0.01
    far = 37
    page, slot = int(table[0, far // block_size]), far % block_size
    kp[page, 0, slot] = 0.0
    kp[page, 0, slot, 3] = 40.0
    q[0, 3] = 40.0
    q[0, head_dim + 3] = 40.0
    got, want = _run_attention(ops, q, kp, vp, cu, ctx, table, q_heads=2, kv_heads=1, head_dim=head_dim)
    torch.testing.assert_close(got, want, **tol(dtype))
    torch.testing.assert_close(got[0, :head_dim], vp[page, 0, :, slot].float(), **tol(dtype))


def test_argmax_rows(ops):
    g = torch.Generator().manual_seed(10)
    logits = rand(g, 5, 1003)
    logits[1, 17] = logits[1, 900] = 50.0          # tie: lowest index
    logits[2, 5] = float("nan")
    logits[3, :] = float("-inf")
    logits[4, 7] = float("inf")
    tokens = torch.zeros(5, dtype=torch.int32, device=DEV)
    status = torch.zeros(5, dtype=torch.int32, device=DEV)
    ops.argmax_rows(logits.to(DEV), tokens, status)
    assert tokens.cpu()[0] == logits[0].argmax() and tokens.cpu()[1] == 17
    assert status.cpu().tolist() == [0, 0, 1, 4, 2]


def sample_params(ops, rows):
    return ops.pack_sample_params(rows).to(DEV)


def test_sampling_follows_the_distribution(ops):
    vocab, draws = 37, 4000
    g = torch.Generator().manual_seed(11)
    row = rand(g, vocab, scale=2.0)
    row[5] = float("-inf")
    logits = row.repeat(draws, 1).to(DEV)
    params = sample_params(ops, [(0.8, None, 1.0, 0.0, 1234, i) for i in range(draws)])
    tokens = torch.zeros(draws, dtype=torch.int32, device=DEV)
    status = torch.zeros(draws, dtype=torch.int32, device=DEV)
    ops.sample_filtered_rows(logits, params, tokens, status)
    assert int(status.sum()) == 0
    got = tokens.cpu()
    # same uniforms, float64 inverse CDF: equal except where the target sits within rounding of a boundary
    want = torch.zeros(draws, dtype=torch.int32)
    refs.sample_filtered_rows(logits.cpu(), params.cpu(), want, torch.zeros(draws, dtype=torch.int32))
    assert (got != want).sum() <= 2
    assert (got == 5).sum() == 0
    probs = torch.softmax(row / 0.8, 0)
    counts = torch.bincount(got.long(), minlength=vocab).float()
    expected = probs * draws
    mask = expected > 5
    chi2 = (((counts - expected) ** 2 / expected)[mask]).sum()
    assert chi2 < 2.0 * int(mask.sum()) + 20
    # a second run with the same seeds and counters repeats the draws; another seed does not
    again = torch.zeros_like(tokens)
    ops.sample_filtered_rows(logits, params, again, status)
    assert torch.equal(again.cpu(), got)
    ops.sample_filtered_rows(logits, sample_params(ops, [(0.8, None, 1.0, 0.0, 1235, i) for i in range(draws)]), again, status)
    assert not torch.equal(again.cpu(), got)


def test_sampling_at_low_temperature_is_argmax(ops):
    g = torch.Generator().manual_seed(12)
    logits = rand(g, 8, 1003).to(DEV)
    tokens = torch.zeros(8, dtype=torch.int32, device=DEV)
    status = torch.zeros(8, dtype=torch.int32, device=DEV)
    ops.sample_filtered_rows(logits, sample_params(ops, [(1e-4, None, 1.0, 0.0, r, 0) for r in range(8)]), tokens, status)
    assert torch.equal(tokens.cpu().long(), logits.cpu().argmax(-1))


FILTERS = [(0.7, 5, 1.0, 0.0), (1.3, None, 0.6, 0.0), (0.9, None, 1.0, 0.1), (0.5, 20, 0.8, 0.05), (1.0, 1, 1.0, 0.0),
           (1.1, 300, 0.95, 0.0), (0.8, None, 0.999, 0.001), (2.0, 50, 0.3, 0.0)]


@pytest.mark.parametrize("vocab,blocks", [(37, 1024), (1003, 1024), (4097, 1024), (151936, 1024), (151936, 100000),
                                          (20000, 100000), (9000, 100000)])
def test_sampling_filters_keep_what_the_reference_keeps(ops, monkeypatch, vocab, blocks):
    """Rows of their own parameters in one call (greedy ones among them), a row in 1, 2, 4, 5 or 32
    slices: every draw equals the float64 inverse CDF over what the reference's filters keep, with
    the same uniform, but for a few whose target lies within rounding of a boundary; a kept set that
    differed by one token would shift every draw behind it."""
    monkeypatch.setattr(ops, "SAMPLE_TARGET_BLOCKS", blocks)
    g = torch.Generator().manual_seed(vocab)
    shapes = FILTERS + [(0.0, None, 1.0, 0.0)]
    per = 24 if vocab > 10000 else 120
    rows, base = [], []
    for f, (t, k, p, m) in enumerate(shapes):
        row = rand(g, vocab, scale=3.0)
        if vocab > 50:
            row[7] = float("-inf")
        for d in range(per):
            rows.append((t, k, p, m, 1000 + f, d))
            base.append(row)
    logits = torch.stack(base)
    wide = torch.full((len(rows), vocab + 3), 9.0)          # rows that are a view with a longer stride
    wide[:, :vocab] = logits
    tokens = torch.zeros(len(rows), dtype=torch.int32, device=DEV)
    status = torch.ones(len(rows), dtype=torch.int32, device=DEV)
    params = sample_params(ops, rows)
    ops.sample_filtered_rows(wide.to(DEV)[:, :vocab], params, tokens, status)
    assert int(status.sum()) == 0
    want = torch.zeros(len(rows), dtype=torch.int32)
    refs.sample_filtered_rows(logits, params.cpu(), want, torch.zeros(len(rows), dtype=torch.int32))
    got = tokens.cpu()
    assert (got != want).sum() <= max(2, len(rows) // 200), (got != want).nonzero().flatten().tolist()
    for f, (t, k, p, m) in enumerate(shapes):       # nothing outside what the filters keep is ever drawn
        picks = got[f * per:(f + 1) * per].long()
        if t == 0.0:
            assert (picks == int(base[f * per].argmax())).all()
            continue
        _, kept = refs.kept_after_filters(base[f * per], t, k or 0, p, m)
        assert kept[picks].all()
    again = torch.zeros_like(tokens)
    ops.sample_filtered_rows(wide.to(DEV)[:, :vocab], params, again, status)
    assert torch.equal(again.cpu(), got)


def test_sampling_thresholds_at_equal_and_extreme_logits(ops):
    """Equal logits (every key in one bin down to the last level), a far maximum (all mass in one
    token), and -inf everywhere but two entries: the searches end and the draws stay inside."""
    vocab = 5000
    flat = torch.zeros(vocab)
    peak = torch.full((vocab,), -50.0)
    peak[4321] = 30.0
    two = torch.full((vocab,), float("-inf"))
    two[17], two[4000] = 1.0, 1.0
    cases = [(flat, (1.0, 10, 0.5, 0.0)), (flat, (1.0, None, 0.5, 0.2)), (peak, (1.0, 40, 0.9, 0.0)), (peak, (5.0, None, 0.99, 0.0)),
             (two, (1.0, 5, 0.9, 0.1)), (two, (0.7, None, 0.4, 0.0))]
    per = 64
    rows = [(t, k, p, m, 7 + c, d) for c, (_, (t, k, p, m)) in enumerate(cases) for d in range(per)]
    logits = torch.stack([row for row, _ in cases for _ in range(per)]).to(DEV)
    tokens = torch.zeros(len(rows), dtype=torch.int32, device=DEV)
    status = torch.ones(len(rows), dtype=torch.int32, device=DEV)
    ops.sample_filtered_rows(logits, sample_params(ops, rows), tokens, status)
    assert int(status.sum()) == 0
    got = tokens.cpu().view(len(cases), per)
    assert len(set(got[0].tolist())) > 20 and len(set(got[1].tolist())) > 20     # equal logits: ties all stay
    assert (got[2] == 4321).all() and (got[3] == 4321).all()
    for c in (4, 5):
        assert set(got[c].tolist()) <= {17, 4000}
    assert set(got[4].tolist()) == {17, 4000}          # top_p 0.9 keeps both halves
    assert set(got[5].tolist()) == {17, 4000}          # equal keys stay together: ties are kept


def test_sampling_reports_bad_rows(ops):
    logits = torch.zeros(4, 100)
    logits[1, 3] = float("nan")
    logits[2, 5] = float("inf")
    logits[3] = float("-inf")
    tokens = torch.zeros(4, dtype=torch.int32, device=DEV)
    status = torch.zeros(4, dtype=torch.int32, device=DEV)
    ops.sample_filtered_rows(logits.to(DEV), sample_params(ops, [(0.9, 5, 0.9, 0.0, 1, 0)] * 4), tokens, status)
    assert status.cpu().tolist() == [0, 1, 2, 4]
    # told that no row limits by top-k or top-p, the call leaves out those launches: the row that does is not through
    ops.sample_filtered_rows(logits.to(DEV), sample_params(ops, [(0.9, 5, 0.9, 0.0, 1, 0)] * 4), tokens, status,
                             any_top_k=False, any_top_p=False)
    assert status.cpu().tolist() == [8, 1, 2, 4]
    with pytest.raises(ops.KernelError):
        ops.sample_filtered_rows(logits.to(DEV), sample_params(ops, [(0.9, 5, 0.9, 0.0, 1, 0)] * 3), tokens, status)


def test_kernels_refuse_what_they_cannot_do(ops):
    from forge_engine_amd.kernels.ops import KernelError
    with pytest.raises(KernelError, match="GPU"):
        ops.swiglu(torch.zeros(2, 8), torch.zeros(2, 4))
    for head_dim in (5, 258):       # odd, or beyond the largest head
        q = torch.zeros(1, head_dim, device=DEV)
        pages = torch.zeros(2, 1, 4, head_dim, device=DEV)
        with pytest.raises(KernelError, match="head size"):
            ops.paged_attention(q, pages, pages.transpose(2, 3).contiguous(), torch.zeros(1, head_dim, device=DEV),
                                torch.tensor([0, 1], dtype=torch.int32, device=DEV),
                                torch.tensor([1], dtype=torch.int32, device=DEV),
                                torch.zeros(1, 1, dtype=torch.int32, device=DEV), num_seqs=1, max_q_len=1,
                                q_heads=1, kv_heads=1, head_dim=head_dim, scale=1.0)


@pytest.mark.parametrize("m", [1, 8, 16, 17, 33, 64])
@pytest.mark.parametrize("n,k", [(64, 8), (200, 200), (1003, 328), (2560, 2560), (330, 9728), (6144, 264)])
def test_gemm_skinny_store(ops, m, n, k):
    g = torch.Generator().manual_seed(20)
    x = rand(g, m, k, dtype=torch.bfloat16)
    w = rand(g, n, k, dtype=torch.bfloat16, scale=0.05)
    want = x.float() @ w.float().T
    got32 = ops.gemm_skinny(x.to(DEV), w.to(DEV), "f32").cpu()
    bound = 2e-6 * float(want.abs().max()) * math.sqrt(k) + 1e-6
    assert float((got32 - want).abs().max()) <= bound
    got16 = ops.gemm_skinny(x.to(DEV), w.to(DEV), "bf16").cpu()
    torch.testing.assert_close(got16.float(), want, atol=1e-2 * float(want.abs().max()), rtol=1e-2)
    # the same call again gives the same bits; a row does not depend on the rows beside it
    assert torch.equal(ops.gemm_skinny(x.to(DEV), w.to(DEV), "f32").cpu(), got32)
    alone = ops.gemm_skinny(x[:1].contiguous().to(DEV), w.to(DEV), "f32").cpu()
    if m <= 16:       # up to 16 rows share one kernel shape: bit-equal; beyond, equal up to the order of the sums
        assert torch.equal(alone[0], got32[0])
    assert float((alone[0] - got32[0]).abs().max()) <= bound


@pytest.mark.parametrize("m", [1, 8, 40, 64])
@pytest.mark.parametrize("inter,k", [(64, 64), (328, 200), (9728, 2560), (100, 1024)])
def test_gemm_skinny_swiglu(ops, m, inter, k):
    g = torch.Generator().manual_seed(21)
    x = rand(g, m, k, dtype=torch.bfloat16)
    w = rand(g, 2 * inter, k, dtype=torch.bfloat16, scale=0.05)
    want = refs.linear_swiglu(x, w).float()
    got = ops.gemm_skinny(x.to(DEV), w.to(DEV), "swiglu").cpu().float()
    torch.testing.assert_close(got, want, atol=1e-2 * float(want.abs().max()) + 1e-6, rtol=1e-2)
    routed = ops.linear_swiglu(x.to(DEV), w.to(DEV)).cpu().float()
    if m <= 16 and k % 64:       # up to 16 rows where the product that pairs gate and up rows does not fit: this kernel
        assert torch.equal(routed, got)
    torch.testing.assert_close(routed, want, atol=1e-2 * float(want.abs().max()) + 1e-6, rtol=1e-2)


@pytest.mark.parametrize("m", [1, 5, 16])
@pytest.mark.parametrize("n,k", [(8200, 264), (9003, 1000), (8209, 2560), (8195, 4096), (8200, 5120), (8209, 6144), (8195, 4104)])
def test_gemm_skinny_resident(ops, m, n, k):
    """Weights with more than 512 row tiles take the variant whose blocks stay and keep x in
    registers: same bits as the one-tile-per-block kernel with as many waves a block (8 up to
    K = 4096, 16 beyond), also for the gated product."""
    g = torch.Generator().manual_seed(23)
    x = rand(g, m, k, dtype=torch.bfloat16).to(DEV)
    w = rand(g, n, k, dtype=torch.bfloat16, scale=0.05).to(DEV)
    want = x.float().cpu() @ w.float().cpu().T
    waves = 8 if k <= 4096 else 16
    plain = ops.gemm_skinny(x, w, "f32", tiles=1, waves=waves).cpu()
    bound = 2e-6 * float(want.abs().max()) * math.sqrt(k) + 1e-6
    assert float((plain - want).abs().max()) <= bound
    assert torch.equal(ops.gemm_skinny(x, w, "f32", tiles=-1).cpu(), plain)
    assert torch.equal(ops.gemm_skinny(x, w, "f32").cpu(), plain)
    assert torch.equal(ops.gemm_skinny(x, w, "bf16").cpu(), ops.gemm_skinny(x, w, "bf16", tiles=1, waves=waves).cpu())
    if n % 2:
        w = w[:n - 1]
    gated = ops.gemm_skinny(x, w, "swiglu", tiles=-1).cpu()
    assert torch.equal(gated, ops.gemm_skinny(x, w, "swiglu", tiles=1, waves=waves).cpu())
    want = refs.linear_swiglu(x.cpu(), w.cpu()).float()
    torch.testing.assert_close(gated.float(), want, atol=1e-2 * float(want.abs().max()) + 1e-6, rtol=1e-2)


def test_gemm_skinny_resident_refuses(ops):
    from forge_engine_amd.kernels.ops import KernelError
    x = torch.zeros(17, 64, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(64, 64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(KernelError):
        ops.gemm_skinny(x, w, "f32", tiles=-1)          # more than 16 rows
    x = torch.zeros(4, 6152, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(64, 6152, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(KernelError):
        ops.gemm_skinny(x, w, "f32", tiles=-1)          # K beyond what the registers hold


@pytest.mark.parametrize("m,n,k,splits", [(1, 200, 1000, 3), (8, 2560, 9728, 4), (16, 330, 4096, 16), (5, 64, 264, 2)])
def test_gemm_skinny_parts_and_their_consumers(ops, m, n, k, splits):
    """K summed in parts by blocks of their own: the parts add up to the product, and the norm and
    the plain add take them as they are (added in order, so repeated calls give the same bits)."""
    g = torch.Generator().manual_seed(24)
    x = rand(g, m, k, dtype=torch.bfloat16).to(DEV)
    w = rand(g, n, k, dtype=torch.bfloat16, scale=0.05).to(DEV)
    whole = ops.gemm_skinny(x, w, "f32", tiles=1, waves=8)
    parts = ops.gemm_skinny(x, w, "f32", tiles=1, waves=8, splits=splits)
    assert parts.shape == (splits, m, n)
    want = x.float().cpu() @ w.float().cpu().T
    bound = 2e-6 * float(want.abs().max()) * math.sqrt(k) + 1e-6
    assert float((parts.sum(0).cpu() - want).abs().max()) <= bound
    assert float((whole.cpu() - want).abs().max()) <= bound
    h = rand(g, m, n).to(DEV)
    nw = rand(g, n).to(DEV)
    summed = parts[0].clone()
    for part in parts[1:]:
        summed += part
    for dtype in (torch.float32, torch.bfloat16):
        h1, h2 = h.clone(), h.clone()
        got = ops.add_rmsnorm(h1, parts, nw, 1e-6, torch.empty(m, n, dtype=dtype, device=DEV))
        ref = ops.add_rmsnorm(h2, summed, nw, 1e-6, torch.empty(m, n, dtype=dtype, device=DEV))
        assert torch.equal(got, ref) and torch.equal(h1, h2)
    h1, h2 = h.clone(), h.clone()
    assert torch.equal(ops.add_rows(h1, parts), ops.add_rows(h2, summed))
    with pytest.raises(ops.KernelError):
        ops.add_rows(h1, parts[:, :, :-1].contiguous())


def test_linear_update_routes(ops):
    g = torch.Generator().manual_seed(25)
    x = rand(g, 8, 4096, dtype=torch.bfloat16).to(DEV)
    few_rows = rand(g, 320, 4096, dtype=torch.bfloat16, scale=0.05).to(DEV)
    many_rows = rand(g, 8192, 4096, dtype=torch.bfloat16, scale=0.05).to(DEV)
    assert ops.linear_update(x, few_rows).dim() == 3              # few row tiles, long K: parts
    assert ops.linear_update(x[:3].contiguous(), many_rows).dim() == 2     # many row tiles, up to three rows: K whole
    tall = ops.linear_update(x, many_rows)                        # four to 16 rows through a weight of many rows: the product for portions
    assert tall.dim() == 3
    torch.testing.assert_close(tall.sum(0).cpu(), x.float().cpu() @ many_rows.float().cpu().T, atol=2e-3, rtol=2e-3)
    x12 = rand(g, 12, 4096, dtype=torch.bfloat16).to(DEV)         # nine to 16 rows: the same whatever the weight
    torch.testing.assert_close(ops.linear_update(x12, few_rows).sum(0).cpu(), x12.float().cpu() @ few_rows.float().cpu().T, atol=2e-3, rtol=2e-3)
    assert ops.linear_update(x[:3, :1024].contiguous(), few_rows[:, :1024]).dim() == 2      # a short K, up to three rows: K whole
    short = ops.linear_update(x[:, :1024].contiguous(), few_rows[:, :1024])
    torch.testing.assert_close((short.sum(0) if short.dim() == 3 else short).cpu(),
                               x[:, :1024].float().cpu() @ few_rows[:, :1024].float().cpu().T, atol=1e-3, rtol=1e-3)
    big = rand(g, 70, 4096, dtype=torch.bfloat16).to(DEV)
    assert ops.linear_update(big, few_rows).shape[1:] == (70, 320)     # 65 to 384 rows: the product for portions, in parts
    huge = rand(g, 500, 4096, dtype=torch.bfloat16).to(DEV)
    assert ops.linear_update(huge, few_rows).shape == (500, 320)       # beyond: the library
    want = x.float().cpu() @ few_rows.float().cpu().T
    torch.testing.assert_close(ops.linear_update(x, few_rows).sum(0).cpu(), want, atol=1e-3, rtol=1e-3)


@pytest.mark.parametrize("m", [17, 33, 48, 64, 5])
@pytest.mark.parametrize("n,k,parts", [(2560, 4096, 8), (2560, 9728, 9), (200, 256, 2), (1003, 1024, 3), (64, 128, 1), (70, 640, 5),
                                       (330, 1408, 2), (96, 2048, 16), (40, 896, 1)])
def test_gemm_mid_parts(ops, m, n, k, parts):
    """17 to 64 rows: K in parts over blocks of 64 weight rows, x staged through LDS; the parts add
    up to the product, each row independent of the rows beside it, the same bits every time."""
    g = torch.Generator().manual_seed(26)
    x = rand(g, m, k, dtype=torch.bfloat16).to(DEV)
    w = rand(g, n, k, dtype=torch.bfloat16, scale=0.05).to(DEV)
    got = ops.gemm_mid_parts(x, w, parts)
    assert got.shape == (parts, m, n)
    want = x.float().cpu() @ w.float().cpu().T
    bound = 2e-6 * float(want.abs().max()) * math.sqrt(k) + 1e-6
    assert float((got.sum(0).cpu() - want).abs().max()) <= bound
    assert torch.equal(ops.gemm_mid_parts(x, w, parts), got)
    alone = ops.gemm_mid_parts(x[2:3].contiguous(), w, parts)
    assert torch.equal(alone[:, 0], got[:, 2])
    # a padded weight (row stride beyond K) and what the residual stream does with the parts
    wide = torch.zeros(n, k + 8, dtype=torch.bfloat16, device=DEV)
    wide[:, :k] = w
    assert torch.equal(ops.gemm_mid_parts(x, wide[:, :k], parts), got)
    h = rand(g, m, n).to(DEV)
    h1, h2 = h.clone(), h.clone()
    summed = got[0].clone()
    for part in got[1:]:
        summed += part
    assert torch.equal(ops.add_rows(h1, got), ops.add_rows(h2, summed))


@pytest.mark.parametrize("m", [17, 33, 64, 65, 100, 128, 130, 300])
@pytest.mark.parametrize("n,k,parts", [(2560, 4096, 8), (200, 256, 2), (1003, 1024, 3), (64, 64, 1), (70, 640, 5), (330, 9728, 16)])
@pytest.mark.parametrize("row_tile", [16, 32, 64, 128])
def test_gemm_wide_parts(ops, m, n, k, parts, row_tile):
    """The product for portions of prompts: partial sums over parts of K (parts without steps are
    zeros), any number of rows in tiles of 64 or 128, weight rows that are no multiple of the
    block's 64, a weight that is a view with a longer row stride."""
    g = torch.Generator().manual_seed(m + n + k)
    x = rand(g, m, k, dtype=torch.bfloat16)
    w_full = rand(g, n, k + 8, dtype=torch.bfloat16, scale=0.05)
    w = w_full[:, :k]
    got = ops.gemm_wide(x.to(DEV), w_full.to(DEV)[:, :k], "parts", parts, row_tile, {100: 32, 130: 128, 300: 128}.get(m, 64))
    assert got.shape == (parts, m, n)
    want = x.float() @ w.float().t()
    torch.testing.assert_close(got.sum(0).cpu(), want, atol=1e-3 * (k / 256) ** 0.5, rtol=1e-3)
    steps = k // 64
    per = -(-steps // parts)
    for part in range(parts):
        lo, hi = part * per * 64, min(k, (part + 1) * per * 64)
        want_part = x[:, lo:hi].float() @ w[:, lo:hi].float().t() if lo < hi else torch.zeros(m, n)
        torch.testing.assert_close(got[part].cpu(), want_part, atol=1e-3 * (k / 256) ** 0.5, rtol=1e-3)


@pytest.mark.parametrize("m", [9, 16, 20, 64, 77, 256, 260])
@pytest.mark.parametrize("n,k", [(6144, 2560), (200, 192), (1002, 320)])
def test_gemm_wide_stores_and_gates(ops, m, n, k):
    g = torch.Generator().manual_seed(m * 3 + n + k)
    x = rand(g, m, k, dtype=torch.bfloat16)
    w = rand(g, n, k, dtype=torch.bfloat16, scale=0.05)
    want = x.float() @ w.float().t()
    for row_tile, block_rows in ((64, 64), (128, 64), (64, 32), (128, 32)):      # blocks of four waves or two
        got = ops.gemm_wide(x.to(DEV), w.to(DEV), "bf16", 1, row_tile, block_rows)
        torch.testing.assert_close(got.cpu().float(), want.to(torch.bfloat16).float(), atol=2e-2, rtol=2e-2)
        gated = ops.gemm_wide(x.to(DEV), w.to(DEV), "swiglu", 1, row_tile, block_rows)
        gate, up = want[:, :n // 2], want[:, n // 2:]
        torch.testing.assert_close(gated.cpu().float(), (gate / (1 + torch.exp(-gate)) * up), atol=2e-2, rtol=2e-2)
        assert gated.shape == (m, n // 2)
    # the ending that takes 8 gate rows and their 8 up rows a wave, blocks of four to eight waves
    for width in (32, 40, 48, 56, 64):
        gated = ops.gemm_wide(x.to(DEV), w.to(DEV), "swiglu_half", 1, 64 if width != 48 else 128, width)
        torch.testing.assert_close(gated.cpu().float(), (gate / (1 + torch.exp(-gate)) * up), atol=2e-2, rtol=2e-2)
    # tiles of 16 and 32 rows (what few rows take): the plain stores and the half-tile gate ending
    for row_tile, width in ((16, 40), (32, 64), (16, 32)):
        got = ops.gemm_wide(x.to(DEV), w.to(DEV), "bf16", 1, row_tile, 64 if width != 32 else 32)
        torch.testing.assert_close(got.cpu().float(), want.to(torch.bfloat16).float(), atol=2e-2, rtol=2e-2)
        gated = ops.gemm_wide(x.to(DEV), w.to(DEV), "swiglu_half", 1, row_tile, width)
        torch.testing.assert_close(gated.cpu().float(), (gate / (1 + torch.exp(-gate)) * up), atol=2e-2, rtol=2e-2)
    with pytest.raises(ops.KernelError):
        ops.gemm_wide(x.to(DEV), w.to(DEV), "swiglu", 1, 16, 64)        # the two-tile gate ending takes tiles of 64 and 128 rows


@pytest.mark.parametrize("shape", [0, 1, 2, 3])
@pytest.mark.parametrize("m", [1, 70, 256, 300, 513])
@pytest.mark.parametrize("inter,k", [(9728, 2560), (200, 192), (1003, 320), (64, 64)])
def test_gemm_gated_tile(ops, shape, m, inter, k):
    """The gate/up product with its SwiGLU ending for any number of rows (tiles of 128 or 256 rows of x
    in LDS, 64 or 128 output columns a block): row counts and widths that are no multiple of the tile,
    a width that is odd (the rows of the result then leave element by element), one step of K."""
    g = torch.Generator().manual_seed(70 + shape)
    x = rand(g, m, k, dtype=torch.bfloat16)
    w = rand(g, 2 * inter, k, dtype=torch.bfloat16, scale=0.05)
    want = refs.linear_swiglu(x, w).float()
    got = ops.gemm_gated(x.to(DEV), w.to(DEV), shape).cpu()
    assert got.shape == (m, inter) and got.dtype == torch.bfloat16
    torch.testing.assert_close(got.float(), want, atol=2e-2 * float(want.abs().max()), rtol=2e-2)
    # a weight whose rows lie further apart than they are long (a slice of a wider matrix)
    wide = rand(g, 2 * inter, k + 64, dtype=torch.bfloat16, scale=0.05).to(DEV)
    view = wide[:, :k]
    want = refs.linear_swiglu(x, view.cpu()).float()
    torch.testing.assert_close(ops.gemm_gated(x.to(DEV), view, shape).cpu().float(), want,
                               atol=2e-2 * float(want.abs().max()), rtol=2e-2)


def test_gemm_gated_tile_refuses(ops):
    g = torch.Generator().manual_seed(71)
    x = rand(g, 8, 96, dtype=torch.bfloat16).to(DEV)                 # K no multiple of 64
    with pytest.raises(ops.KernelError):
        ops.gemm_gated(x, rand(g, 64, 96, dtype=torch.bfloat16).to(DEV))
    x = rand(g, 8, 128, dtype=torch.bfloat16).to(DEV)
    with pytest.raises(ops.KernelError):
        ops.gemm_gated(x, rand(g, 63, 128, dtype=torch.bfloat16).to(DEV))      # an odd number of weight rows
    with pytest.raises(ops.KernelError):
        ops.gemm_gated(x, rand(g, 64, 128, dtype=torch.bfloat16).to(DEV), shape=7)
    with pytest.raises(ops.KernelError):
        ops.gemm_gated(x.float(), rand(g, 64, 128, dtype=torch.bfloat16).to(DEV))


def test_linear_swiglu_routes_by_rows(ops, monkeypatch):
    """Up to 64 rows at a K of up to 3072: the product that pairs gate and up rows within a wave (at a
    longer K from 17 rows, the streaming kernel below); more: the matrix library and the gate kernel.
    All give the plain result."""
    g = torch.Generator().manual_seed(33)
    w = rand(g, 2 * 328, 256, dtype=torch.bfloat16, scale=0.05)
    taken = []
    real_call = ops._call
    monkeypatch.setattr(ops, "_call", lambda lib, name, *a: taken.append(name) or real_call(lib, name, *a))
    for rows, name in ((1, "fe_gemm_wide"), (8, "fe_gemm_wide"), (17, "fe_gemm_wide"), (64, "fe_gemm_wide"), (65, "fe_swiglu")):
        x = rand(g, rows, 256, dtype=torch.bfloat16)
        taken.clear()
        got = ops.linear_swiglu(x.to(DEV), w.to(DEV)).cpu().float()
        assert taken[-1] == name, taken
        y = x.float() @ w.float().t()
        gate, up = y[:, :328], y[:, 328:]
        torch.testing.assert_close(got, gate / (1 + torch.exp(-gate)) * up, atol=2e-2, rtol=2e-2)
    assert ops._gate_block_columns(9728) == 40 and ops._gate_block_columns(12288) == 48
    # a K of 4096: the streaming kernel up to 16 rows, the paired product from 17
    mid_k = rand(g, 2 * 40, 4096, dtype=torch.bfloat16, scale=0.02)
    for rows, name in ((8, "fe_gemm_skinny"), (16, "fe_gemm_skinny"), (17, "fe_gemm_wide")):
        x = rand(g, rows, 4096, dtype=torch.bfloat16)
        taken.clear()
        got = ops.linear_swiglu(x.to(DEV), mid_k.to(DEV)).cpu().float()
        assert taken[-1] == name, (rows, taken)
        y = x.float() @ mid_k.float().t()
        torch.testing.assert_close(got, y[:, :40] / (1 + torch.exp(-y[:, :40])) * y[:, 40:], atol=2e-2, rtol=2e-2)
    # a K beyond the one up to which that product wins: the library and the gate kernel at 17 to 64 rows too
    long_k = rand(g, 2 * 40, 5120, dtype=torch.bfloat16, scale=0.02)
    x = rand(g, 32, 5120, dtype=torch.bfloat16)
    taken.clear()
    got = ops.linear_swiglu(x.to(DEV), long_k.to(DEV)).cpu().float()
    assert taken[-1] == "fe_swiglu", taken
    y = x.float() @ long_k.float().t()
    torch.testing.assert_close(got, y[:, :40] / (1 + torch.exp(-y[:, :40])) * y[:, 40:], atol=2e-2, rtol=2e-2)
    # 2,048 to 4,096 rows at a K of up to 3,072: the product that keeps tiles of x in LDS and forms the ending itself
    for rows, k, name in ((2047, 256, "fe_swiglu"), (2048, 256, "fe_gemm_gated"), (4096, 256, "fe_gemm_gated"), (4097, 256, "fe_swiglu"),
                          (2048, 4096, "fe_swiglu")):
        weight = rand(g, 2 * 72, k, dtype=torch.bfloat16, scale=0.05)
        x = rand(g, rows, k, dtype=torch.bfloat16)
        taken.clear()
        got = ops.linear_swiglu(x.to(DEV), weight.to(DEV)).cpu().float()
        assert taken[-1] == name, (rows, k, taken)
        torch.testing.assert_close(got, refs.linear_swiglu(x, weight).float(), atol=2e-2, rtol=2e-2)


def test_gemm_wide_refuses_and_routes(ops, monkeypatch):
    x = torch.zeros(70, 200, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(64, 200, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ops.KernelError):
        ops.gemm_wide(x, w, "parts", 2)                    # K is no multiple of 64
    with pytest.raises(ops.KernelError):
        ops.gemm_wide(x[:, :192].contiguous(), w[:, :192], "bf16", 2)     # a stored product has one part
    taken = []
    real_call = ops._call
    monkeypatch.setattr(ops, "_call", lambda lib, name, *a: taken.append(name) or real_call(lib, name, *a))
    g = torch.Generator().manual_seed(5)
    x = rand(g, 100, 256, dtype=torch.bfloat16).to(DEV)
    w = rand(g, 320, 256, dtype=torch.bfloat16, scale=0.05).to(DEV)
    update = ops.linear_update(x, w, None, torch.zeros(100, 320, device=DEV))
    assert update is not None and update.dim() == 3 and taken == ["fe_gemm_wide"]
    torch.testing.assert_close(update.sum(0).cpu(), x.float().cpu() @ w.float().cpu().t(), atol=1e-3, rtol=1e-3)
    y = ops.linear(x, w)
    assert taken == ["fe_gemm_wide"] and y.dtype == torch.bfloat16      # 100 rows x 320 weight rows: too few blocks, the library's
    wide = rand(g, 4544, 256, dtype=torch.bfloat16, scale=0.05).to(DEV)  # 71 blocks of 64 weight rows x 2 row tiles: its own
    y = ops.linear(x, wide)
    assert taken == ["fe_gemm_wide", "fe_gemm_wide"] and y.shape == (100, 4544)
    torch.testing.assert_close(y.float().cpu(), x.float().cpu() @ wide.float().cpu().t(), atol=2e-2, rtol=2e-2)
    y = ops.linear(x[:64], w)
    assert taken == ["fe_gemm_wide"] * 3                                 # up to 64 rows it takes any weight that fits
    torch.testing.assert_close(y.float().cpu(), x[:64].float().cpu() @ w.float().cpu().t(), atol=2e-2, rtol=2e-2)
    big = rand(g, 600, 256, dtype=torch.bfloat16).to(DEV)
    assert ops.linear_update(big, w, None, torch.zeros(600, 320, device=DEV)) is None and len(taken) == 3   # the library's


def test_gemm_mid_parts_refuses_a_k_that_is_no_multiple_of_its_step(ops):
    g = torch.Generator().manual_seed(27)
    x = rand(g, 20, 264, dtype=torch.bfloat16).to(DEV)
    w = rand(g, 100, 264, dtype=torch.bfloat16).to(DEV)
    with pytest.raises(ops.KernelError):
        ops.gemm_mid_parts(x, w, 2)
    update = ops.linear_update(x, w)                      # the library takes it
    assert update.shape == (20, 100)
    torch.testing.assert_close(update.cpu(), x.float().cpu() @ w.float().cpu().T, atol=1e-3, rtol=1e-3)


def test_linear_update_adds_into_the_stream_where_the_library_multiplies(ops):
    """More than 64 rows: the matrix library's product adds into the float32 stream as it stores and
    nothing is left pending; the stream then holds exactly stream + product.  Fewer rows: the update
    comes back (in parts) and the stream is left alone."""
    g = torch.Generator().manual_seed(31)
    for m, n, k in ((500, 320, 256), (390, 2560, 4096)):
        x, w = rand(g, m, k, dtype=torch.bfloat16).to(DEV), rand(g, n, k, dtype=torch.bfloat16, scale=0.05).to(DEV)
        stream = rand(g, m, n).to(DEV)
        before = stream.clone()
        assert ops.linear_update(x, w, None, stream) is None
        want = before + ops.linear_update(x, w)
        assert torch.equal(stream, want)
        torch.testing.assert_close(stream.cpu(), before.cpu() + x.float().cpu() @ w.float().cpu().t(), atol=2e-3, rtol=2e-3)
    x, w = rand(g, 8, 256, dtype=torch.bfloat16).to(DEV), rand(g, 320, 256, dtype=torch.bfloat16).to(DEV)
    stream = rand(g, 8, 320).to(DEV)
    before = stream.clone()
    assert ops.linear_update(x, w, None, stream) is not None and torch.equal(stream, before)


def test_linear_update_is_in_parts_from_17_rows(ops, monkeypatch):
    taken = []
    real_call = ops._call
    monkeypatch.setattr(ops, "_call", lambda lib, name, *a: taken.append(name) or real_call(lib, name, *a))
    g = torch.Generator().manual_seed(27)
    w = rand(g, 2560, 4096, dtype=torch.bfloat16, scale=0.05).to(DEV)
    for rows in (17, 40, 64):
        x = rand(g, rows, 4096, dtype=torch.bfloat16).to(DEV)
        update = ops.linear_update(x, w)
        assert update.dim() == 3 and update.shape[1:] == (rows, 2560)
        assert update.shape[0] == 6 and taken[-1] == "fe_gemm_wide"      # 40 blocks a part: six parts fill 240 CUs
        want = x.float().cpu() @ w.float().cpu().T
        torch.testing.assert_close(update.sum(0).cpu(), want, atol=2e-3, rtol=2e-3)
    more = rand(g, 65, 4096, dtype=torch.bfloat16).to(DEV)          # 65 rows and more: the same product, tiles of 128 rows
    update = ops.linear_update(more, w)
    assert update.dim() == 3 and taken[-1] == "fe_gemm_wide"
    torch.testing.assert_close(update.sum(0).cpu(), more.float().cpu() @ w.float().cpu().T, atol=2e-3, rtol=2e-3)
    assert ops.linear_update(rand(g, 400, 4096, dtype=torch.bfloat16).to(DEV), w).dim() == 2     # the library
    # a weight of more rows than the product for portions takes: the product for 17 to 64 rows
    tall = rand(g, 8256, 1024, dtype=torch.bfloat16, scale=0.05).to(DEV)
    x = rand(g, 40, 1024, dtype=torch.bfloat16).to(DEV)
    update = ops.linear_update(x, tall)
    assert update.dim() == 3 and taken[-1] == "fe_gemm_mid_parts"
    torch.testing.assert_close(update.sum(0).cpu(), x.float().cpu() @ tall.float().cpu().T, atol=2e-3, rtol=2e-3)


def test_linear_routes_by_rows_and_dtype(ops):
    g = torch.Generator().manual_seed(22)
    w = rand(g, 136, 200, dtype=torch.bfloat16, scale=0.05)
    for rows in (3, 64, 65, 300):     # up to 64 rows: the streaming kernel; beyond: the matrix library
        x = rand(g, rows, 200, dtype=torch.bfloat16)
        want = x.float() @ w.float().T
        got = ops.linear(x.to(DEV), w.to(DEV), out_dtype=torch.float32).cpu()
        torch.testing.assert_close(got, want, atol=1e-3, rtol=1e-3)
        assert ops.linear(x.to(DEV), w.to(DEV)).dtype == torch.bfloat16
    # a weight stored in 32-bit stays in 32-bit: the activation is widened
    got = ops.linear(x.to(DEV), w.float().to(DEV)).cpu()
    assert got.dtype == torch.bfloat16
    torch.testing.assert_close(got.float(), want, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("splits", [1, 3, 8])
@pytest.mark.parametrize("q_heads,kv_heads,head_dim,block_size", [
    (32, 8, 128, 16), (5, 5, 64, 16), (10, 2, 128, 32), (8, 1, 256, 16), (6, 3, 64, 64), (16, 2, 128, 16),
])
def test_decode_attention_kernel(ops, q_heads, kv_heads, head_dim, block_size, splits):
    """The streaming decode kernel (single-token sequences of a bfloat16 cache) with key splits;
    sequences with more tokens in the same batch go to the general kernel."""
    g = torch.Generator().manual_seed(30)
    seqs = [(0, 1), (14, 1), (15, 1), (16, 1), (699, 1), (40, 6), (255, 1), (3, 1)]
    q, kp, vp, cu, ctx, table = _attention_case(g, torch.bfloat16, seqs, q_heads, kv_heads, head_dim, block_size,
                                                extra_width=2 * kv_heads * head_dim)
    kw = dict(num_seqs=len(seqs), max_q_len=6, q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim,
              scale=head_dim ** -0.5)
    want = refs.paged_attention(q, kp, vp, torch.empty(q.shape[0], q_heads * head_dim, dtype=q.dtype), cu, ctx, table, **kw).float()
    got = ops.paged_attention(q.to(DEV), kp.to(DEV), vp.to(DEV),
                              torch.full((q.shape[0], q_heads * head_dim), float("nan"), dtype=q.dtype, device=DEV),
                              cu.to(DEV), ctx.to(DEV), table.to(DEV), num_decode=7, max_ctx=700, splits=splits, **kw).cpu().float()
    torch.testing.assert_close(got, want, atol=2e-2, rtol=2e-2)
    # the splits' arrival counters are left at zero: further launches (other values, same pages) agree too
    dev = [t.to(DEV) for t in (kp, vp, cu, ctx, table)]
    for factor in (0.5, -2.0, 1.0):
        out = torch.full((q.shape[0], q_heads * head_dim), float("nan"), dtype=q.dtype, device=DEV)
        again = ops.paged_attention((q * factor).to(DEV), dev[0], dev[1], out, dev[2], dev[3], dev[4],
                                    num_decode=7, max_ctx=700, splits=splits, **kw).cpu().float()
        if factor == 1.0:
            assert torch.equal(again, got)
        else:
            expect = refs.paged_attention(q * factor, kp, vp, torch.empty(q.shape[0], q_heads * head_dim, dtype=q.dtype),
                                          cu, ctx, table, **kw).float()
            torch.testing.assert_close(again, expect, atol=2e-2, rtol=2e-2)


LONG_CONTEXTS = [2046, 4095, 19999, 33, 0, 700, 8191]     # tokens each sequence holds before its one new token


@pytest.mark.parametrize("q_heads,kv_heads,head_dim,block_size", [(4, 2, 128, 16), (5, 1, 64, 32)])
def test_decode_attention_kernel_every_count_of_key_splits(ops, q_heads, kv_heads, head_dim, block_size):
    """Every count of key splits that the kernel takes (1 to 64: the merges with all loads in one
    round for up to 4, 8 and 16 splits, and the loop beyond), over contexts from one key to 20,000:
    splits without any key, splits of one 32-key block, a context one short of a block's and a
    page's edge.  Each count is launched twice on the same arrival counters, with other queries."""
    g = torch.Generator().manual_seed(61)
    seqs = [(before, 1) for before in LONG_CONTEXTS]
    q, kp, vp, cu, ctx, table = _attention_case(g, torch.bfloat16, seqs, q_heads, kv_heads, head_dim, block_size,
                                                extra_width=2 * kv_heads * head_dim)
    kw = dict(q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim, scale=head_dim ** -0.5)
    queries = [q, (q.float() * -1.5).to(torch.bfloat16)]
    wants = [refs.paged_attention_by_matrices(x, kp, vp, cu, ctx, table, **kw) for x in queries]
    dev = [t.to(DEV) for t in (kp, vp, cu, ctx, table)]
    queries_dev = [x.to(DEV) for x in queries]
    assert set(refs.DECODE_SPLITS_TESTED) == set(range(1, 65))
    for splits in refs.DECODE_SPLITS_TESTED:
        for x, want in zip(queries_dev, wants):
            out = torch.full((len(seqs), q_heads * head_dim), float("nan"), dtype=torch.bfloat16, device=DEV)
            ops.paged_attention(x, dev[0], dev[1], out, dev[2], dev[3], dev[4], num_seqs=len(seqs), max_q_len=1,
                                num_decode=len(seqs), max_ctx=20000, splits=splits, **kw)
            torch.testing.assert_close(out.cpu().float(), want, atol=2e-2, rtol=2e-2, msg=lambda m: f"{splits} splits: {m}")


@pytest.mark.parametrize("splits", [9, 12, 16, 17, 32, 64])
@pytest.mark.parametrize("q_heads,kv_heads,head_dim,block_size", [(4, 2, 128, 16), (8, 1, 64, 32)])
def test_decode_attention_that_prepares_with_many_key_splits(ops, q_heads, kv_heads, head_dim, block_size, splits):
    """The kernel that makes its own queries and keys with 9 to 64 key splits over long contexts,
    against the plain reference of the two steps; twice on the same pages and counters."""
    g = torch.Generator().manual_seed(62)
    qkv, kp, vp, cu, ctx, table, qw, kw, inv_freq, positions, token_seq = _prepare_case(
        g, q_heads, kv_heads, head_dim, block_size, LONG_CONTEXTS)
    n = len(LONG_CONTEXTS)
    sizes = dict(q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim)
    qkv_ref, kp_ref, vp_ref = qkv.clone(), kp.clone(), vp.clone()
    refs.qk_norm_rope_write(qkv_ref, qw, kw, inv_freq, positions, token_seq, table, kp_ref, vp_ref,
                            rotary_dim=head_dim, eps=1e-6, **sizes)
    want = refs.paged_attention_by_matrices(qkv_ref, kp_ref, vp_ref, cu, ctx, table, scale=head_dim ** -0.5, **sizes)
    kp_dev, vp_dev = kp.to(DEV), vp.to(DEV)
    for _ in range(2):
        out = torch.full((n, q_heads * head_dim), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.decode_attention_prepare(qkv.to(DEV), qw.to(DEV), kw.to(DEV), inv_freq.to(DEV), kp_dev, vp_dev, out, cu.to(DEV),
                                     ctx.to(DEV), table.to(DEV), eps=1e-6, scale=head_dim ** -0.5, max_ctx=20000,
                                     splits=splits, **sizes)
        torch.testing.assert_close(out.cpu().float(), want, atol=2e-2, rtol=2e-2)
    torch.testing.assert_close(kp_dev.cpu().float(), kp_ref.float(), **tol(torch.bfloat16))
    assert torch.equal(vp_dev.cpu(), vp_ref)


@pytest.mark.parametrize("batch,kv_heads,context,chosen", [(1, 8, 2048, 16), (1, 8, 8192, 32), (1, 1, 16384, 64), (2, 8, 2048, 16)])
def test_decode_attention_with_the_key_splits_that_the_step_chooses(ops, batch, kv_heads, context, chosen):
    """What a decode step at batch 1 or 2 launches once its block tables are wider than 64 pages:
    the count of key splits is left to ``ops.decode_splits`` (given the table-width bound as the
    step gives it), both for finished queries and for the kernel that prepares its own."""
    assert ops.decode_splits(batch, kv_heads, context) == chosen
    g = torch.Generator().manual_seed(63)
    q_heads, head_dim, block_size = 2 * kv_heads, 64, 16
    contexts = [context - 1 - 37 * i for i in range(batch)]     # the longest fills the bound to its last key
    qkv, kp, vp, cu, ctx, table, qw, kw, inv_freq, positions, token_seq = _prepare_case(
        g, q_heads, kv_heads, head_dim, block_size, contexts)
    sizes = dict(q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim)
    qkv_ref, kp_ref, vp_ref = qkv.clone(), kp.clone(), vp.clone()
    refs.qk_norm_rope_write(qkv_ref, qw, kw, inv_freq, positions, token_seq, table, kp_ref, vp_ref,
                            rotary_dim=head_dim, eps=1e-6, **sizes)
    want = refs.paged_attention_by_matrices(qkv_ref, kp_ref, vp_ref, cu, ctx, table, scale=head_dim ** -0.5, **sizes)
    out = torch.full((batch, q_heads * head_dim), float("nan"), dtype=torch.bfloat16, device=DEV)
    kp_dev, vp_dev = kp.to(DEV), vp.to(DEV)
    ops.decode_attention_prepare(qkv.to(DEV), qw.to(DEV), kw.to(DEV), inv_freq.to(DEV), kp_dev, vp_dev, out, cu.to(DEV),
                                 ctx.to(DEV), table.to(DEV), eps=1e-6, scale=head_dim ** -0.5, max_ctx=context, **sizes)
    torch.testing.assert_close(out.cpu().float(), want, atol=2e-2, rtol=2e-2)
    # finished queries over the pages that the launch above completed
    out = torch.full((batch, q_heads * head_dim), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.paged_attention(qkv_ref.to(DEV), kp_dev, vp_dev, out, cu.to(DEV), ctx.to(DEV), table.to(DEV), num_seqs=batch,
                        max_q_len=1, num_decode=batch, max_ctx=context, scale=head_dim ** -0.5, **sizes)
    torch.testing.assert_close(out.cpu().float(), want, atol=2e-2, rtol=2e-2)


def test_attention_kernels_on_random_mixed_batches(ops):
    """Random head counts, groups, page sizes, windows and mixtures of single tokens and portions
    (with and without context before them): the fast kernels that a bfloat16 batch is routed to
    against the plain reference."""
    import random
    rng = random.Random(77)
    for case in range(24):
        head_dim = rng.choice([64, 128])
        kv_heads = rng.choice([1, 2, 3])
        groups = rng.choice([1, 2, 4, 5, 8])
        q_heads = kv_heads * groups
        block_size = rng.choice([16, 32, 64])
        window = rng.choice([None, None, 1, 17, 64, 100])
        seqs = [(rng.choice([0, 0, 1, 15, 16, 63, 64, rng.randrange(0, 300)]),
                 rng.choice([1, 1, 2, 3, 17, 63, 64, 65, 130, rng.randrange(2, 200)])) for _ in range(rng.randrange(1, 5))]
        g = torch.Generator().manual_seed(100 + case)
        q, kp, vp, cu, ctx, table = _attention_case(g, torch.bfloat16, seqs, q_heads, kv_heads, head_dim, block_size,
                                                    extra_width=2 * kv_heads * head_dim)
        kw = dict(num_seqs=len(seqs), max_q_len=max(n for _, n in seqs), q_heads=q_heads, kv_heads=kv_heads,
                  head_dim=head_dim, scale=head_dim ** -0.5, window=window)
        want = refs.paged_attention(q, kp, vp, torch.empty(q.shape[0], q_heads * head_dim, dtype=q.dtype), cu, ctx, table, **kw).float()
        got = ops.paged_attention(q.to(DEV), kp.to(DEV), vp.to(DEV),
                                  torch.full((q.shape[0], q_heads * head_dim), float("nan"), dtype=q.dtype, device=DEV),
                                  cu.to(DEV), ctx.to(DEV), table.to(DEV), num_decode=sum(1 for _, n in seqs if n == 1),
                                  max_ctx=max(b + n for b, n in seqs), **kw).cpu().float()
        assert torch.isfinite(got).all(), (case, seqs)
        torch.testing.assert_close(got, want, atol=2e-2, rtol=2e-2, msg=lambda m: f"case {case} {seqs} window {window}: {m}")


def _prepare_case(g, q_heads, kv_heads, head_dim, block_size, contexts):
    """A step of single tokens: raw projection output, norm weights, frequencies, filled pages."""
    seqs = [(before, 1) for before in contexts]
    qkv, kp, vp, cu, ctx, table = _attention_case(g, torch.bfloat16, seqs, q_heads, kv_heads, head_dim, block_size,
                                                  extra_width=2 * kv_heads * head_dim)
    qw, kw = 1.0 + rand(g, head_dim, scale=0.1), 1.0 + rand(g, head_dim, scale=0.1)
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    positions = torch.tensor(contexts, dtype=torch.int32)
    token_seq = torch.arange(len(contexts), dtype=torch.int32)
    return qkv, kp, vp, cu, ctx, table, qw, kw, inv_freq, positions, token_seq


@pytest.mark.parametrize("splits", [1, 3, 8])
@pytest.mark.parametrize("with_norm", [True, False])
@pytest.mark.parametrize("q_heads,kv_heads,head_dim,block_size", [
    (32, 8, 128, 16), (5, 5, 64, 16), (10, 2, 128, 32), (8, 1, 256, 16), (6, 3, 64, 64), (7, 1, 128, 16),
])
def test_decode_attention_that_prepares_its_queries_and_keys(ops, q_heads, kv_heads, head_dim, block_size, splits, with_norm):
    """One launch from the projection's output to the attention's output against the plain
    reference of the two steps (norm + rotation + cache write, then attention), and against the
    two kernels that do the same in two launches: the pages must hold the same bits."""
    g = torch.Generator().manual_seed(33)
    contexts = [0, 1, 14, 15, 16, 31, 32, 699, 255, 3]      # tokens each sequence holds before the step
    qkv, kp, vp, cu, ctx, table, qw, kw, inv_freq, positions, token_seq = _prepare_case(
        g, q_heads, kv_heads, head_dim, block_size, contexts)
    if not with_norm:
        qw = kw = None
    n = len(contexts)
    sizes = dict(q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim)
    akw = dict(num_seqs=n, max_q_len=1, scale=head_dim ** -0.5, **sizes)
    # plain reference
    qkv_ref, kp_ref, vp_ref = qkv.clone(), kp.clone(), vp.clone()
    refs.qk_norm_rope_write(qkv_ref, qw, kw, inv_freq, positions, token_seq, table, kp_ref, vp_ref,
                            rotary_dim=head_dim, eps=1e-6, **sizes)
    want = refs.paged_attention(qkv_ref, kp_ref, vp_ref, torch.empty(n, q_heads * head_dim, dtype=qkv.dtype),
                                cu, ctx, table, **akw).float()
    # two launches
    dev = lambda t: None if t is None else t.to(DEV)
    qkv_two, kp_two, vp_two = qkv.to(DEV), kp.to(DEV), vp.to(DEV)
    ops.qk_norm_rope_write(qkv_two, dev(qw), dev(kw), dev(inv_freq), dev(positions), dev(token_seq), dev(table),
                           kp_two, vp_two, rotary_dim=head_dim, eps=1e-6, **sizes)
    two = ops.paged_attention(qkv_two, kp_two, vp_two, torch.empty(n, q_heads * head_dim, dtype=qkv.dtype, device=DEV),
                              dev(cu), dev(ctx), dev(table), num_decode=n, max_ctx=700, splits=splits, **akw).cpu().float()
    # one launch, twice (the second on the pages the first left: the arrival counters are zero again)
    qkv_one, kp_one, vp_one = qkv.to(DEV), kp.to(DEV), vp.to(DEV)
    for _ in range(2):
        out = torch.full((n, q_heads * head_dim), float("nan"), dtype=qkv.dtype, device=DEV)
        ops.decode_attention_prepare(qkv_one, dev(qw), dev(kw), dev(inv_freq), kp_one, vp_one, out, dev(cu), dev(ctx),
                                     dev(table), eps=1e-6, scale=head_dim ** -0.5, max_ctx=700, splits=splits, **sizes)
        got = out.cpu().float()
        assert torch.equal(qkv_one.cpu(), qkv)               # the projection's output is left alone
        assert torch.equal(kp_one.cpu(), kp_two.cpu())       # same bits as the stand-alone kernel writes
        assert torch.equal(vp_one.cpu(), vp_two.cpu())
        torch.testing.assert_close(got, want, atol=2e-2, rtol=2e-2)
        torch.testing.assert_close(got, two, atol=2e-2, rtol=2e-2)
    torch.testing.assert_close(kp_one.cpu().float(), kp_ref.float(), **tol(torch.bfloat16))
    assert torch.equal(vp_one.cpu(), vp_ref)


@pytest.mark.parametrize("parts", [1, 2, 3, 4])
@pytest.mark.parametrize("q_heads,kv_heads,head_dim,block_size", [(32, 8, 128, 16), (5, 5, 64, 32), (8, 1, 256, 16)])
def test_decode_attention_that_prepares_from_partial_sums(ops, q_heads, kv_heads, head_dim, block_size, parts):
    """The projection's output as float32 partial sums: added up in order and rounded to bfloat16
    inside the kernel, after which everything is as with the rounded matrix as input (same
    output, same bits in the pages)."""
    g = torch.Generator().manual_seed(37)
    contexts = [0, 15, 16, 300, 77]
    qkv, kp, vp, cu, ctx, table, qw, kw, inv_freq, _, _ = _prepare_case(g, q_heads, kv_heads, head_dim, block_size, contexts)
    n = len(contexts)
    sums = rand(g, parts, n, qkv.shape[1])
    total = sums[0].clone()
    for part in sums[1:]:
        total += part
    rounded = total.to(torch.bfloat16)
    sizes = dict(q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim)
    results = []
    for source in (rounded, sums):
        kp_dev, vp_dev, src = kp.to(DEV), vp.to(DEV), source.to(DEV)
        out = torch.full((n, q_heads * head_dim), float("nan"), dtype=torch.bfloat16, device=DEV)
        for splits in (1, 3):
            ops.decode_attention_prepare(src, qw.to(DEV), kw.to(DEV), inv_freq.to(DEV), kp_dev, vp_dev, out, cu.to(DEV),
                                         ctx.to(DEV), table.to(DEV), eps=1e-6, scale=head_dim ** -0.5, max_ctx=301,
                                         splits=splits, **sizes)
        assert torch.equal(src.cpu(), source)
        results.append((out.cpu(), kp_dev.cpu(), vp_dev.cpu()))
    for a, b in zip(*results):
        assert torch.equal(a, b)
    with pytest.raises(ops.KernelError):
        ops.decode_attention_prepare(rand(g, 5, n, qkv.shape[1]).to(DEV), qw.to(DEV), kw.to(DEV), inv_freq.to(DEV), kp.to(DEV),
                                     vp.to(DEV), torch.empty(n, q_heads * head_dim, dtype=torch.bfloat16, device=DEV), cu.to(DEV),
                                     ctx.to(DEV), table.to(DEV), eps=1e-6, scale=1.0, **sizes)


def test_linear_in_parts(ops):
    g = torch.Generator().manual_seed(38)
    w = rand(g, 6144, 2560, dtype=torch.bfloat16, scale=0.05).to(DEV)
    for rows in (1, 8, 16, 17, 64):
        x = rand(g, rows, 2560, dtype=torch.bfloat16).to(DEV)
        sums = ops.linear_in_parts(x, w)
        assert sums.dtype == torch.float32 and sums.dim() == 3 and sums.shape[0] <= 4 and sums.shape[1:] == (rows, 6144)
        torch.testing.assert_close(sums.sum(0).cpu(), x.cpu().float() @ w.cpu().float().T, atol=2e-3, rtol=2e-3)
    assert ops.linear_in_parts(rand(g, 65, 2560, dtype=torch.bfloat16).to(DEV), w) is None       # many rows: the library
    assert ops.linear_in_parts(rand(g, 4, 256, dtype=torch.bfloat16).to(DEV), w[:, :256]) is None  # a short K
    assert ops.linear_in_parts(rand(g, 4, 2560).to(DEV), w.float()) is None                        # not bfloat16


@pytest.mark.parametrize("window", [1, 16, 37, 300])
def test_decode_attention_that_prepares_with_a_window(ops, window):
    g = torch.Generator().manual_seed(34)
    contexts = [0, 36, 37, 500]
    qkv, kp, vp, cu, ctx, table, qw, kw, inv_freq, positions, token_seq = _prepare_case(g, 8, 2, 128, 16, contexts)
    sizes = dict(q_heads=8, kv_heads=2, head_dim=128)
    qkv_ref, kp_ref, vp_ref = qkv.clone(), kp.clone(), vp.clone()
    refs.qk_norm_rope_write(qkv_ref, qw, kw, inv_freq, positions, token_seq, table, kp_ref, vp_ref,
                            rotary_dim=128, eps=1e-5, **sizes)
    want = refs.paged_attention(qkv_ref, kp_ref, vp_ref, torch.empty(4, 1024, dtype=qkv.dtype), cu, ctx, table,
                                num_seqs=4, max_q_len=1, scale=0.1, window=window, **sizes).float()
    for splits in (1, 4):
        kp_dev, vp_dev = kp.to(DEV), vp.to(DEV)
        out = torch.full((4, 1024), float("nan"), dtype=qkv.dtype, device=DEV)
        ops.decode_attention_prepare(qkv.to(DEV), qw.to(DEV), kw.to(DEV), inv_freq.to(DEV), kp_dev, vp_dev, out,
                                     cu.to(DEV), ctx.to(DEV), table.to(DEV), eps=1e-5, scale=0.1, window=window,
                                     max_ctx=501, splits=splits, **sizes)
        torch.testing.assert_close(out.cpu().float(), want, atol=2e-2, rtol=2e-2)
        assert torch.equal(vp_dev.cpu(), vp_ref)


def test_decode_attention_that_prepares_sees_its_own_token_and_a_far_key(ops):
    """The new token's own key never comes from memory, and keys far back do: each made to
    stand out in turn (query and key are unit vectors scaled up, no norm, position 0 rotation
    aside the rotation keeps lengths, so q.k of the chosen pair dominates)."""
    g = torch.Generator().manual_seed(35)
    head_dim, block_size, before = 128, 16, 999
    qkv, kp, vp, cu, ctx, table, _, _, inv_freq, positions, token_seq = _prepare_case(g, 4, 1, head_dim, block_size, [before])
    qkv = (qkv.float() * 0.01).to(torch.bfloat16)
    sizes = dict(q_heads=4, kv_heads=1, head_dim=head_dim)
    # its own token: the new key is the query's direction, scaled up; rotation by the same angle keeps q.k
    own = qkv.clone()
    own[0, :5 * head_dim] = 0.0
    for h in range(5):                       # four query heads and the key head
        own[0, h * head_dim + 5] = 30.0
    for splits in (1, 5):
        kp_dev, vp_dev = kp.to(DEV), vp.to(DEV)
        out = torch.empty(1, 4 * head_dim, dtype=qkv.dtype, device=DEV)
        ops.decode_attention_prepare(own.to(DEV), None, None, inv_freq.to(DEV), kp_dev, vp_dev, out, cu.to(DEV),
                                     ctx.to(DEV), table.to(DEV), eps=1e-6, scale=head_dim ** -0.5, max_ctx=1000,
                                     splits=splits, **sizes)
        new_value = own[0, 5 * head_dim:6 * head_dim].float()
        for h in range(4):
            torch.testing.assert_close(out.cpu().float()[0, h * head_dim:(h + 1) * head_dim], new_value, atol=2e-2, rtol=2e-2)
        page, slot = int(table[0, before // block_size]), before % block_size
        assert torch.equal(vp_dev.cpu()[page, 0, :, slot], own[0, 5 * head_dim:6 * head_dim])
    # a far key: stored as the query's rotated direction (the reference rotates the query for us)
    rotated = own.clone()
    refs.qk_norm_rope_write(rotated, None, None, inv_freq, positions, token_seq, table, kp.clone(), vp.clone(),
                            rotary_dim=head_dim, eps=1e-6, **sizes)
    quiet = own.clone()
    quiet[0, 4 * head_dim:5 * head_dim] = 0.0            # the new key says nothing
    for far in (0, 15, 16, 511, 512, 991, 998):
        kq = kp.clone()
        page, slot = int(table[0, far // block_size]), far % block_size
        kq[page, 0, slot] = rotated[0, :head_dim]
        for splits in (1, 5):
            out = torch.empty(1, 4 * head_dim, dtype=qkv.dtype, device=DEV)
            ops.decode_attention_prepare(quiet.to(DEV), None, None, inv_freq.to(DEV), kq.to(DEV), vp.to(DEV), out,
                                         cu.to(DEV), ctx.to(DEV), table.to(DEV), eps=1e-6, scale=head_dim ** -0.5,
                                         max_ctx=1000, splits=splits, **sizes)
            for h in range(4):
                torch.testing.assert_close(out.cpu().float()[0, h * head_dim:(h + 1) * head_dim],
                                           vp[page, 0, :, slot].float(), atol=2e-2, rtol=2e-2)


def test_decode_attention_that_prepares_refuses_what_it_does_not_serve(ops):
    g = torch.Generator().manual_seed(36)
    qkv, kp, vp, cu, ctx, table, qw, kw, inv_freq, _, _ = _prepare_case(g, 4, 2, 64, 16, [3, 9])
    dev = lambda t: t.to(DEV)
    out = torch.empty(2, 256, dtype=torch.bfloat16, device=DEV)
    call = lambda **over: ops.decode_attention_prepare(
        **{**dict(qkv=dev(qkv), q_weight=dev(qw), k_weight=dev(kw), inv_freq=dev(inv_freq), key_pages=dev(kp),
                  value_pages=dev(vp), out=out, cu_q=dev(cu), ctx_len=dev(ctx), block_table=dev(table), q_heads=4,
                  kv_heads=2, head_dim=64, eps=1e-6, scale=0.125), **over})
    call()
    with pytest.raises(ops.KernelError):
        call(inv_freq=dev(inv_freq[:16]))                  # a head rotated in part
    with pytest.raises(ops.KernelError):
        call(k_weight=None)                                # one norm without the other
    with pytest.raises(ops.KernelError):
        call(qkv=dev(qkv[:, :-64].contiguous()))           # no room for the values
    assert not ops.decode_prepare_supported(torch.float32, q_heads=4, kv_heads=2, head_dim=64, rotary_dim=64, block_size=16)
    assert not ops.decode_prepare_supported(torch.bfloat16, q_heads=4, kv_heads=2, head_dim=48, rotary_dim=48, block_size=16)
    assert not ops.decode_prepare_supported(torch.bfloat16, q_heads=18, kv_heads=2, head_dim=64, rotary_dim=64, block_size=16)


@pytest.mark.parametrize("window", [1, 16, 37, 300])
def test_decode_attention_kernel_window(ops, window):
    g = torch.Generator().manual_seed(31)
    seqs = [(0, 1), (36, 1), (37, 1), (500, 1)]
    q, kp, vp, cu, ctx, table = _attention_case(g, torch.bfloat16, seqs, 8, 2, 128, 16)
    kw = dict(num_seqs=4, max_q_len=1, q_heads=8, kv_heads=2, head_dim=128, scale=128 ** -0.5, window=window)
    want = refs.paged_attention(q, kp, vp, torch.empty(4, 1024, dtype=q.dtype), cu, ctx, table, **kw).float()
    for splits in (1, 4):
        got = ops.paged_attention(q.to(DEV), kp.to(DEV), vp.to(DEV), torch.empty(4, 1024, dtype=q.dtype, device=DEV),
                                  cu.to(DEV), ctx.to(DEV), table.to(DEV), num_decode=4, max_ctx=501, splits=splits, **kw).cpu().float()
        torch.testing.assert_close(got, want, atol=2e-2, rtol=2e-2)


def test_decode_attention_far_key_and_page_edges(ops):
    """One key far back, and keys at the first and last slot of a page, each made to stand out in turn."""
    g = torch.Generator().manual_seed(32)
    head_dim, block_size, ctx_len = 128, 16, 1000
    q, kp, vp, cu, ctx, table = _attention_case(g, torch.bfloat16, [(ctx_len - 1, 1)], 4, 1, head_dim, block_size)
    q = (q.float() * 0.01).to(torch.bfloat16)
    for far in (0, 15, 16, 37, 511, 512, 991, 999):
        kq, qq = kp.clone(), q.clone()
        page, slot = int(table[0, far // block_size]), far % block_size
        kq[page, 0, slot] = 0.0
        kq[page, 0, slot, 5] = 30.0
        for h in range(4):
            qq[0, h * head_dim + 5] = 30.0
        for splits in (1, 5):
            got = ops.paged_attention(qq.to(DEV), kq.to(DEV), vp.to(DEV), torch.empty(1, 4 * head_dim, dtype=q.dtype, device=DEV),
                                      cu.to(DEV), ctx.to(DEV), table.to(DEV), num_seqs=1, max_q_len=1, q_heads=4, kv_heads=1,
                                      head_dim=head_dim, scale=head_dim ** -0.5, num_decode=1, max_ctx=ctx_len, splits=splits).cpu().float()
            for h in range(4):
                torch.testing.assert_close(got[0, h * head_dim:(h + 1) * head_dim], vp[page, 0, :, slot].float(), atol=2e-2, rtol=2e-2)


def _poison_unowned_slots(kp, vp, table, owned_from, owned_to, block_size):
    """NaN into every slot of the pages that no live key owns: whole pages outside the tables,
    slots at or beyond a sequence's context, slots below its window.  owned_from/to: per sequence."""
    owned = torch.zeros(kp.shape[0], block_size, dtype=torch.bool)
    for s in range(table.shape[0]):
        for key in range(owned_from[s], owned_to[s]):
            owned[int(table[s, key // block_size]), key % block_size] = True
    kp[~owned[:, None, :, None].expand_as(kp)] = float("nan")
    vp[~owned[:, None, None, :].expand_as(vp)] = float("nan")


@pytest.mark.parametrize("window", [None, 40])
def test_attention_kernels_ignore_what_unowned_slots_hold(ops, window):
    """A page that is leased again still holds what the request before left there, which may be a
    NaN (a batch that overflowed).  Every slot that no live key of the batch owns is set to NaN:
    the fast kernels (single tokens with and without key splits, portions) must give what they
    give for clean pages.  With a window, the slots below it count as unowned too and their table
    entries are -1, as the cache manager leaves them once the window has passed."""
    g = torch.Generator().manual_seed(43)
    q_heads, kv_heads, head_dim, block_size = 8, 2, 128, 16
    seqs = [(0, 70), (100, 1), (13, 9), (129, 1), (3, 1), (60, 66), (0, 2), (31, 1)]
    q, kp, vp, cu, ctx, table = _attention_case(g, torch.bfloat16, seqs, q_heads, kv_heads, head_dim, block_size,
                                                extra_width=2 * kv_heads * head_dim)
    kw = dict(num_seqs=len(seqs), max_q_len=70, q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim,
              scale=head_dim ** -0.5, window=window)
    want = refs.paged_attention(q, kp, vp, torch.empty(q.shape[0], q_heads * head_dim, dtype=q.dtype), cu, ctx, table, **kw).float()
    first = [0 if window is None else max(0, before - window + 1) for before, _ in seqs]
    kp_bad, vp_bad, table_bad = kp.clone(), vp.clone(), table.clone()
    _poison_unowned_slots(kp_bad, vp_bad, table, first, [b + n for b, n in seqs], block_size)
    for s, low in enumerate(first):
        table_bad[s, :low // block_size] = -1               # pages wholly below the window were given back
    assert torch.isnan(kp_bad).any() and torch.isnan(vp_bad).any()
    for splits in (1, 3):
        got = ops.paged_attention(q.to(DEV), kp_bad.to(DEV), vp_bad.to(DEV),
                                  torch.full((q.shape[0], q_heads * head_dim), float("nan"), dtype=q.dtype, device=DEV),
                                  cu.to(DEV), ctx.to(DEV), table_bad.to(DEV), num_decode=4, max_ctx=130, splits=splits, **kw).cpu().float()
        assert torch.isfinite(got).all()
        torch.testing.assert_close(got, want, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("window", [None, 40])
def test_decode_attention_that_prepares_ignores_what_unowned_slots_hold(ops, window):
    g = torch.Generator().manual_seed(44)
    contexts = [0, 15, 16, 100, 129, 31]
    qkv, kp, vp, cu, ctx, table, qw, kw, inv_freq, positions, token_seq = _prepare_case(g, 8, 2, 128, 16, contexts)
    sizes = dict(q_heads=8, kv_heads=2, head_dim=128)
    qkv_ref, kp_ref, vp_ref = qkv.clone(), kp.clone(), vp.clone()
    refs.qk_norm_rope_write(qkv_ref, qw, kw, inv_freq, positions, token_seq, table, kp_ref, vp_ref,
                            rotary_dim=128, eps=1e-6, **sizes)
    want = refs.paged_attention(qkv_ref, kp_ref, vp_ref, torch.empty(6, 1024, dtype=qkv.dtype), cu, ctx, table,
                                num_seqs=6, max_q_len=1, scale=128 ** -0.5, window=window, **sizes).float()
    first = [0 if window is None else max(0, before - window + 1) for before in contexts]
    table_bad = table.clone()
    for s, low in enumerate(first):
        table_bad[s, :low // 16] = -1
    for splits in (1, 3):
        kp_bad, vp_bad = kp.clone(), vp.clone()
        _poison_unowned_slots(kp_bad, vp_bad, table, first, contexts, 16)   # the new token's slot is unowned before the step
        kp_dev, vp_dev = kp_bad.to(DEV), vp_bad.to(DEV)
        out = torch.full((6, 1024), float("nan"), dtype=qkv.dtype, device=DEV)
        ops.decode_attention_prepare(qkv.to(DEV), qw.to(DEV), kw.to(DEV), inv_freq.to(DEV), kp_dev, vp_dev, out,
                                     cu.to(DEV), ctx.to(DEV), table_bad.to(DEV), eps=1e-6, scale=128 ** -0.5, window=window,
                                     max_ctx=130, splits=splits, **sizes)
        assert torch.isfinite(out).all()
        torch.testing.assert_close(out.cpu().float(), want, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("q_heads,kv_heads,head_dim,block_size", [
    (8, 2, 128, 16), (5, 5, 64, 16), (12, 1, 128, 32), (3, 3, 64, 64),
])
@pytest.mark.parametrize("row_sets", [1, 2])
def test_prefill_attention_kernel(ops, q_heads, kv_heads, head_dim, block_size, row_sets, monkeypatch):
    """The matrix-core kernel for portions of prompts: whole prompts, portions with context already
    cached, lengths that are no multiple of the tile, beside single tokens in the same batch; with
    blocks of 64 and of 128 query rows."""
    monkeypatch.setattr(ops, "PREFILL_ROW_SETS", row_sets)
    g = torch.Generator().manual_seed(40)
    seqs = [(0, 130), (70, 1), (13, 9), (0, 2), (200, 65), (63, 64), (5, 1), (0, 64)]
    q, kp, vp, cu, ctx, table = _attention_case(g, torch.bfloat16, seqs, q_heads, kv_heads, head_dim, block_size,
                                                extra_width=2 * kv_heads * head_dim)
    kw = dict(num_seqs=len(seqs), max_q_len=130, q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim,
              scale=head_dim ** -0.5)
    want = refs.paged_attention(q, kp, vp, torch.empty(q.shape[0], q_heads * head_dim, dtype=q.dtype), cu, ctx, table, **kw).float()
    got = ops.paged_attention(q.to(DEV), kp.to(DEV), vp.to(DEV),
                              torch.full((q.shape[0], q_heads * head_dim), float("nan"), dtype=q.dtype, device=DEV),
                              cu.to(DEV), ctx.to(DEV), table.to(DEV), num_decode=2, max_ctx=265, **kw).cpu().float()
    torch.testing.assert_close(got, want, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("num_seqs", [40, 64, 65, 130])
@pytest.mark.parametrize("row_sets", [1, 2])
def test_prefill_attention_kernel_places_every_tile(ops, num_seqs, row_sets, monkeypatch):
    """The kernel's grid holds a place for every 64-row (or 128-row) tile there may be (the host knows only the
    step's tokens and sequences) and every block finds its sequence and tile on the device: up to 64
    sequences by a search with a lane a sequence, more one after the other.  Sequences of every
    kind side by side: empty ones (a captured step pads with them), single tokens, one to four tiles,
    with and without cached context."""
    monkeypatch.setattr(ops, "PREFILL_ROW_SETS", row_sets)
    g = torch.Generator().manual_seed(50 + num_seqs)
    lengths = torch.randint(0, 7, (num_seqs,), generator=g).tolist()
    seqs = []
    for kind in lengths:
        q_len = {0: 0, 1: 1, 2: 2, 3: 64, 4: 65, 5: 130, 6: 200}[kind]
        before = int(torch.randint(0, 90, (1,), generator=g)) if kind % 2 else 0
        seqs.append((before if q_len else 16, q_len))
    q_heads, kv_heads, head_dim, block_size = 8, 2, 64, 16
    q, kp, vp, cu, ctx, table = _attention_case(g, torch.bfloat16, seqs, q_heads, kv_heads, head_dim, block_size,
                                                extra_width=2 * kv_heads * head_dim)
    kw = dict(num_seqs=len(seqs), max_q_len=200, q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim,
              scale=head_dim ** -0.5)
    want = refs.paged_attention(q, kp, vp, torch.empty(q.shape[0], q_heads * head_dim, dtype=q.dtype), cu, ctx, table, **kw).float()
    got = ops.paged_attention(q.to(DEV), kp.to(DEV), vp.to(DEV),
                              torch.full((q.shape[0], q_heads * head_dim), float("nan"), dtype=q.dtype, device=DEV),
                              cu.to(DEV), ctx.to(DEV), table.to(DEV), num_decode=None, max_ctx=300, **kw).cpu().float()
    assert torch.isfinite(got).all()
    torch.testing.assert_close(got, want, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("window", [None, 100, 700])
@pytest.mark.parametrize("q_heads,kv_heads,head_dim,block_size", [(8, 2, 128, 16), (6, 3, 64, 32)])
@pytest.mark.parametrize("key_groups", [1, 2])
@pytest.mark.parametrize("row_sets", [1, 2])
def test_prefill_attention_kernel_long_walks(ops, q_heads, kv_heads, head_dim, block_size, window, key_groups, row_sets, monkeypatch):
    """Launches that leave the chip underfilled take blocks of two key groups that walk every
    other tile and merge at the end: walks of one tile (the second group idle), of an odd and an
    even number of tiles, behind a long context, beside single tokens; with unowned slots
    poisoned.  Every kind of block (one or two key groups, 64 or 128 rows), forced in turn."""
    monkeypatch.setattr(ops, "PREFILL_KEY_GROUPS", key_groups)
    monkeypatch.setattr(ops, "PREFILL_ROW_SETS", row_sets)
    g = torch.Generator().manual_seed(45)
    seqs = [(0, 300), (500, 257), (70, 1), (3, 2), (1000, 64), (0, 64), (61, 67)]
    q, kp, vp, cu, ctx, table = _attention_case(g, torch.bfloat16, seqs, q_heads, kv_heads, head_dim, block_size,
                                                extra_width=2 * kv_heads * head_dim)
    kw = dict(num_seqs=len(seqs), max_q_len=300, q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim,
              scale=head_dim ** -0.5, window=window)
    want = refs.paged_attention(q, kp, vp, torch.empty(q.shape[0], q_heads * head_dim, dtype=q.dtype), cu, ctx, table, **kw).float()
    first = [0 if window is None else max(0, before - window + 1) for before, _ in seqs]
    _poison_unowned_slots(kp, vp, table, first, [b + n for b, n in seqs], block_size)
    got = ops.paged_attention(q.to(DEV), kp.to(DEV), vp.to(DEV),
                              torch.full((q.shape[0], q_heads * head_dim), float("nan"), dtype=q.dtype, device=DEV),
                              cu.to(DEV), ctx.to(DEV), table.to(DEV), num_decode=1, max_ctx=2048, **kw).cpu().float()
    assert torch.isfinite(got).all()
    torch.testing.assert_close(got, want, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("key_groups", [1, 2])
@pytest.mark.parametrize("row_sets", [1, 2])
@pytest.mark.parametrize("seqs,q_heads,kv_heads,head_dim", [
    ([(0, 2048)], 4, 2, 128), ([(0, 8192)], 2, 1, 128), ([(0, 1024)] * 8, 4, 2, 64), ([(6000, 2048), (0, 1)], 2, 1, 64),
])
def test_prefill_attention_kernel_at_the_lengths_of_the_benchmarks(ops, seqs, q_heads, kv_heads, head_dim, key_groups, row_sets, monkeypatch):
    """Whole prompts of 2,048 and 8,192 tokens, eight of 1,024, and a portion of 2,048 behind 6,000
    cached tokens: walks of up to 128 key tiles, with blocks of one and of two key groups, of 64 and of 128 rows."""
    monkeypatch.setattr(ops, "PREFILL_KEY_GROUPS", key_groups)
    monkeypatch.setattr(ops, "PREFILL_ROW_SETS", row_sets)
    g = torch.Generator().manual_seed(46)
    q, kp, vp, cu, ctx, table = _attention_case(g, torch.bfloat16, seqs, q_heads, kv_heads, head_dim, 16,
                                                extra_width=2 * kv_heads * head_dim)
    kw = dict(q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim, scale=head_dim ** -0.5)
    want = refs.paged_attention_by_matrices(q, kp, vp, cu, ctx, table, **kw)
    longest = max(n for _, n in seqs)
    got = ops.paged_attention(q.to(DEV), kp.to(DEV), vp.to(DEV),
                              torch.full((q.shape[0], q_heads * head_dim), float("nan"), dtype=q.dtype, device=DEV),
                              cu.to(DEV), ctx.to(DEV), table.to(DEV), num_seqs=len(seqs), max_q_len=longest,
                              num_decode=sum(1 for _, n in seqs if n == 1), max_ctx=max(b + n for b, n in seqs), **kw).cpu().float()
    assert torch.isfinite(got).all()
    torch.testing.assert_close(got, want, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("window", [1, 7, 64, 100])
@pytest.mark.parametrize("row_sets", [1, 2])
def test_prefill_attention_kernel_window(ops, window, row_sets, monkeypatch):
    monkeypatch.setattr(ops, "PREFILL_ROW_SETS", row_sets)
    g = torch.Generator().manual_seed(41)
    seqs = [(0, 150), (90, 40), (3, 2)]
    q, kp, vp, cu, ctx, table = _attention_case(g, torch.bfloat16, seqs, 4, 2, 64, 16)
    kw = dict(num_seqs=3, max_q_len=150, q_heads=4, kv_heads=2, head_dim=64, scale=0.125, window=window)
    want = refs.paged_attention(q, kp, vp, torch.empty(q.shape[0], 256, dtype=q.dtype), cu, ctx, table, **kw).float()
    got = ops.paged_attention(q.to(DEV), kp.to(DEV), vp.to(DEV), torch.empty(q.shape[0], 256, dtype=q.dtype, device=DEV),
                              cu.to(DEV), ctx.to(DEV), table.to(DEV), num_decode=0, **kw).cpu().float()
    torch.testing.assert_close(got, want, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("row_sets", [1, 2])
def test_prefill_attention_far_key_and_tile_edges(ops, row_sets, monkeypatch):
    """A query late in a long prompt whose score for one early key stands far out: the key is put at
    the first and last slot of a page and of a 64-key tile in turn."""
    monkeypatch.setattr(ops, "PREFILL_ROW_SETS", row_sets)
    g = torch.Generator().manual_seed(42)
    head_dim, block_size, length = 128, 16, 600
    q, kp, vp, cu, ctx, table = _attention_case(g, torch.bfloat16, [(0, length)], 2, 1, head_dim, block_size)
    q = (q.float() * 0.01).to(torch.bfloat16)
    query = 577
    for far in (0, 15, 16, 63, 64, 127, 128, 300, 575, 576, 577):
        kq, qq = kp.clone(), q.clone()
        page, slot = int(table[0, far // block_size]), far % block_size
        kq[page, 0, slot] = 0.0
        kq[page, 0, slot, 9] = 30.0
        qq[query, 9] = 30.0
        qq[query, head_dim + 9] = 30.0
        got = ops.paged_attention(qq.to(DEV), kq.to(DEV), vp.to(DEV), torch.empty(length, 2 * head_dim, dtype=q.dtype, device=DEV),
                                  cu.to(DEV), ctx.to(DEV), table.to(DEV), num_seqs=1, max_q_len=length, q_heads=2, kv_heads=1,
                                  head_dim=head_dim, scale=head_dim ** -0.5, num_decode=0).cpu().float()
        for h in range(2):
            torch.testing.assert_close(got[query, h * head_dim:(h + 1) * head_dim], vp[page, 0, :, slot].float(), atol=2e-2, rtol=2e-2)
    # a key after the query must stay invisible however large its score would be
    kq = kp.clone()
    page, slot = int(table[0, 578 // block_size]), 578 % block_size
    kq[page, 0, slot, 9] = 100.0
    qq = q.clone()
    qq[query, 9] = 30.0
    got = ops.paged_attention(qq.to(DEV), kq.to(DEV), vp.to(DEV), torch.empty(length, 2 * head_dim, dtype=q.dtype, device=DEV),
                              cu.to(DEV), ctx.to(DEV), table.to(DEV), num_seqs=1, max_q_len=length, q_heads=2, kv_heads=1,
                              head_dim=head_dim, scale=head_dim ** -0.5, num_decode=0).cpu().float()
    assert float((got[query, :head_dim] - vp[page, 0, :, slot].float()).abs().max()) > 0.1
