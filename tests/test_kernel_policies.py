"""Host-side choices of the kernel wrappers that need no GPU: how a product's K is cut into parts
and how many key splits the decode attention takes."""

from __future__ import annotations

import pytest

from forge_engine_amd.kernels import ops


@pytest.mark.parametrize("steps", [1, 3, 4, 7, 20, 32, 76, 500])
@pytest.mark.parametrize("blocks", [1, 3, 40, 96, 160, 1000])
@pytest.mark.parametrize("most", [1, 4, 16])
def test_parts_of_k_are_never_empty_and_respect_their_bounds(steps, blocks, most):
    parts = ops._mid_parts(steps, blocks, most)
    assert 1 <= parts <= most
    per_part = -(-steps // parts)
    assert (parts - 1) * per_part < steps          # the last part still has a step
    assert parts == 1 or per_part >= 4 or steps < 8   # a part is at least four steps long


def test_parts_of_k_for_the_large_model():
    # Qwen3-4B: q/k/v (20 steps, 96 blocks of 64 rows), output (32, 40), down (76, 40)
    assert ops._mid_parts(20, 96, most=4) == 2
    assert ops._mid_parts(32, 40) == 6
    assert ops._mid_parts(76, 40) == 6


@pytest.mark.parametrize("m", [1, 8, 16, 40, 64, 100, 256, 384])
@pytest.mark.parametrize("n", [64, 320, 2560, 4096, 5120, 6144])
@pytest.mark.parametrize("k", [64, 512, 2560, 4096, 9728, 25600])
@pytest.mark.parametrize("block_rows,most", [(64, 16), (32, 4), (128, 16)])
def test_parts_of_the_product_for_portions(m, n, k, block_rows, most):
    parts = ops._wide_parts(m, n, k, block_rows, most)
    steps = k // 64
    assert 1 <= parts <= most
    per_part = -(-steps // parts)
    assert (parts - 1) * per_part < steps                    # no part without steps
    assert parts == 1 or per_part >= 8                       # a part is at least eight 64-steps long


def test_blocks_of_the_products_for_few_rows_fill_the_chip():
    # Qwen3-4B at up to 16 rows: output and down projections in six parts of 40 blocks (240 of 256 CUs)
    assert ops._wide_parts(8, 2560, 4096) == 6 and ops._wide_parts(8, 2560, 9728) == 6
    # q/k/v in blocks of 32 weight rows: 192 blocks a part, four parts (768 = three rounds of 256), never more than
    # the four that the attention launch adds up
    assert ops._wide_parts(8, 6144, 2560, 32, most=4) == 4 and ops._wide_parts(8, 6144, 4096, 32, most=4) == 4
    # Qwen3-8B: 64 blocks a part, four parts fill 256 CUs
    assert ops._wide_parts(8, 4096, 4096) == 4 and ops._wide_parts(8, 4096, 12288) == 4
    # gate/up: columns a block so that the blocks fill rounds of one a CU (9728 / 40 = 244, 12288 / 48 = 256)
    assert ops._gate_block_columns(9728) == 40 and ops._gate_block_columns(12288) == 48


@pytest.mark.parametrize("num_decode,kv_heads,max_ctx,expect", [
    (8, 8, 1040, 4), (1, 8, 2048, 16), (64, 8, 1040, 1), (1, 8, 64, 1), (1, 1, 100000, 64),
])
def test_key_splits_of_the_decode_attention(num_decode, kv_heads, max_ctx, expect):
    assert ops.decode_splits(num_decode, kv_heads, max_ctx) == expect


def test_the_fused_decode_attention_serves_what_it_says():
    import torch
    ok = dict(q_heads=32, kv_heads=8, head_dim=128, rotary_dim=128, block_size=16)
    assert ops.decode_prepare_supported(torch.bfloat16, **ok)
    assert not ops.decode_prepare_supported(torch.float32, **ok)
    for change in (dict(head_dim=96, rotary_dim=96), dict(rotary_dim=64), dict(q_heads=80), dict(block_size=8),
                   dict(block_size=48), dict(q_heads=30)):
        assert not ops.decode_prepare_supported(torch.bfloat16, **{**ok, **change}), change


def test_split_counters_outlive_their_growth():
    """A captured graph keeps the address of the counters it was recorded with: when a step needs
    more of them, the old buffer must stay alive (and zero) beside the new one."""
    import torch

    workspace = ops.Workspace()
    cpu = torch.device("cpu")
    first = workspace.split_counters(cpu, 64)
    address = first.data_ptr()
    assert workspace.split_counters(cpu, 4096) is first           # no growth: the same buffer
    grown = workspace.split_counters(cpu, 100000)
    assert grown.numel() >= 100000 and grown.data_ptr() != address
    assert any(old is first for old in workspace._retired)        # still referenced, so never handed to another tensor
    assert first.data_ptr() == address and int(first.abs().sum()) == 0
    assert workspace.split_counters(cpu, 5000) is grown           # and later launches use the larger one


def test_workspaces_are_per_owner():
    import torch

    a, b = ops.Workspace(), ops.Workspace()
    cpu = torch.device("cpu")
    with ops.use_workspace(a):
        mine = ops._split_counters(cpu, 8)
        with ops.use_workspace(b):
            assert ops._split_counters(cpu, 8) is not mine
        assert ops._split_counters(cpu, 8) is mine
    assert ops._split_counters(cpu, 8) is not mine                # outside: the default of (device, stream)


def test_every_count_of_key_splits_that_a_decode_step_can_take_is_one_that_the_gpu_tests_launch():
    import kernel_refs
    seen = set()
    for batch in list(range(1, 66)) + [96, 128, 255, 256]:
        for kv_heads in (1, 2, 3, 4, 5, 8, 16, 40, 64):
            for ctx in [1, 31, 32, 33, 127, 128, 129] + [64 * n for n in range(1, 1025)]:
                seen.add(ops.decode_splits(batch, kv_heads, ctx))
    assert seen <= set(kernel_refs.DECODE_SPLITS_TESTED)
    assert {1, 16, 17, 64} <= seen and max(seen) == 64 and min(seen) == 1
    # the table-width bound of a captured decode step (a multiple of 64 pages of 16 tokens) at batch 1 and 2 past
    # 1,024 tokens, and at batch 1 past 4,096: the merges of 9 to 16 splits and of 17 to 64
    assert ops.decode_splits(1, 8, 2048) == 16 and ops.decode_splits(2, 8, 2048) == 16
    assert ops.decode_splits(1, 8, 8192) == 32 and ops.decode_splits(1, 1, 16384) == 64


@pytest.mark.parametrize("window", [None, 1, 9, 40])
def test_the_two_references_of_paged_attention_agree(window):
    """The reference by whole matrices (used where sequences are thousands of tokens long) against
    the one that goes token by token: mixed batch, shuffled pages, a window whose passed pages were
    given back."""
    import kernel_refs
    import torch
    g = torch.Generator().manual_seed(5)
    q_heads, kv_heads, head_dim, block_size = 6, 2, 8, 4
    seqs = [(0, 7), (13, 1), (5, 9), (30, 0), (0, 1)]
    total = sum(n for _, n in seqs)
    pages = [-(-(b + n) // block_size) for b, n in seqs]
    order = torch.randperm(sum(pages) + 2, generator=g).tolist()
    table = torch.full((len(seqs), max(pages)), -1, dtype=torch.int32)
    at = 0
    for s, count in enumerate(pages):
        table[s, :count] = torch.tensor(order[at:at + count], dtype=torch.int32)
        at += count
    if window:   # pages that every query's window has passed
        for s, (before, n) in enumerate(seqs):
            table[s, :max(0, before - window + 1) // block_size] = -1
    kp = torch.randn(sum(pages) + 2, kv_heads, block_size, head_dim, generator=g)
    vp = torch.randn(sum(pages) + 2, kv_heads, head_dim, block_size, generator=g)
    q = torch.randn(total, q_heads * head_dim + 5, generator=g)
    cu = torch.tensor([0] + torch.tensor([n for _, n in seqs]).cumsum(0).tolist(), dtype=torch.int32)
    ctx = torch.tensor([b + n for b, n in seqs], dtype=torch.int32)
    kw = dict(q_heads=q_heads, kv_heads=kv_heads, head_dim=head_dim, scale=0.3, window=window)
    slow = kernel_refs.paged_attention(q, kp, vp, torch.empty(total, q_heads * head_dim), cu, ctx, table,
                                       num_seqs=len(seqs), max_q_len=9, **kw)
    fast = kernel_refs.paged_attention_by_matrices(q, kp, vp, cu, ctx, table, **kw)
    torch.testing.assert_close(fast, slow, atol=1e-5, rtol=1e-5)


def test_a_library_that_is_missing_and_cannot_be_built_fails_loudly(monkeypatch, tmp_path):
    """No fallback: without a compiled library and without a compiler, loading raises, and so does
    the preparation of a model's libraries; a file at the library's place that was built from other
    sources is not opened in its stead."""
    from forge_engine_amd.kernels import build, library

    monkeypatch.setattr(build, "library_dirs", lambda: [tmp_path])
    monkeypatch.setattr(library, "_LOADED", {})

    def no_compiler() -> str:
        raise build.KernelBuildError("hipcc not found: the HIP kernels cannot be compiled")

    monkeypatch.setattr(build, "find_hipcc", no_compiler)
    assert not library.is_built("rowwise")
    with pytest.raises(library.KernelUnavailable, match="not built and could not be compiled.*hipcc not found"):
        library.load("rowwise")
    with pytest.raises(library.KernelUnavailable, match="hipcc not found"):
        library.ensure_built(["rowwise", "sample"], announce=False)
    stale = build.library_path("rowwise", tmp_path)
    stale.write_bytes(b"\x7fELF built from sources with another hash")
    assert not library.is_built("rowwise")
    with pytest.raises(library.KernelUnavailable):
        library.load("rowwise")
    assert "rowwise" not in library._LOADED
    with pytest.raises(build.KernelBuildError, match="no kernel source"):
        build.compile_one("no_such_kernel", tmp_path)


def test_operands_on_the_cpu_are_refused_before_anything_is_loaded():
    import torch

    h = torch.zeros(2, 8)
    with pytest.raises(ops.KernelError, match="no CPU path"):
        ops.add_rmsnorm(h, None, torch.ones(8), 1e-6, torch.empty(2, 8))
    with pytest.raises(ops.KernelError, match="no CPU path"):
        ops.linear(torch.zeros(2, 8), torch.zeros(4, 8))


def test_the_product_that_stores_bfloat16_needs_blocks_enough_beyond_64_rows():
    # q/k/v of Qwen3-4B and 8B (6144 weight rows) fill the chip at 65 to 256 rows; of Qwen3-0.6B and 1.7B (4096) they do not
    for rows in (65, 128, 129, 256):
        assert ops._wide_store_pays(rows, 6144) and ops._wide_store_pays(rows, 5120)
        assert not ops._wide_store_pays(rows, 4096) and not ops._wide_store_pays(rows, 2048)
    for rows in (17, 32, 64):
        assert ops._wide_store_pays(rows, 4096, 2048) and ops._wide_store_pays(rows, 7168, 5120)
        assert not ops._wide_store_pays(rows, 8192, 6144)       # 100 MB of weight: the library's
