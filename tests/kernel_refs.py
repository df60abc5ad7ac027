"""Plain PyTorch references of every kernel entry point, with the same
signatures as ``forge_engine_amd.kernels.ops``.

Two uses: the GPU tests compare each HIP kernel alone with its reference here;
the CPU tests patch these in for the kernels (``install``) so that the step
function, the cache and the scheduler can be exercised without a GPU.  They
are test code: the product has no CPU path and never imports this file.
All arithmetic is float32 (float64 where noted), whatever the storage dtype.
"""

from __future__ import annotations

import torch


def embed_rows(ids, table, out):
    out.copy_(table[ids.long()].float())
    return out


def add_rmsnorm(h, delta, weight, eps, out, rows=None, store_sum=True):
    if delta is not None and delta.dim() == 3:
        delta = delta.float().sum(0)
    if rows is not None:
        src = h[rows.long()]
        if delta is not None:
            src = src + delta[rows.long()].float()
    else:
        src = h if delta is None else h + delta.float()
        if delta is not None and store_sum:
            h.copy_(src)
    var = src.square().mean(dim=-1, keepdim=True)
    out.copy_((src * torch.rsqrt(var + eps) * weight).to(out.dtype))
    return out


def add_rows(h, delta):
    h += delta.float().sum(0) if delta.dim() == 3 else delta.float()
    return h


def swiglu(gate_up, out):
    inter = gate_up.shape[1] // 2
    g = gate_up[:, :inter].float()
    u = gate_up[:, inter:].float()
    out.copy_((g / (1.0 + torch.exp(-g)) * u).to(out.dtype))
    return out


def gemm_nt_f32(a, b, bias=None, out=None):
    y = a.double() @ b.double().T
    if bias is not None:
        y = y + bias.double()
    y = y.float()
    if out is None:
        return y
    out.copy_(y)
    return out


def linear(x, weight, bias=None, out_dtype=None):
    y = x.float() @ weight.float().T
    if bias is not None:
        y = y + bias.float()
    return y.to(x.dtype if out_dtype is None else out_dtype)


def linear_swiglu(x, gate_up_weight):
    inter = gate_up_weight.shape[0] // 2
    y = x.float() @ gate_up_weight.float().T
    g, u = y[:, :inter], y[:, inter:]
    return (g / (1.0 + torch.exp(-g)) * u).to(x.dtype)


def linear_update(x, weight, bias=None, stream=None):
    return linear(x, weight, bias, out_dtype=torch.float32)    # the stream is left to the caller's add


def gemm_skinny(x, weight, epilogue="bf16", tiles=0, waves=0, splits=1):
    if epilogue == "swiglu":
        return linear_swiglu(x, weight)
    return linear(x, weight, out_dtype=torch.float32 if epilogue == "f32" else torch.bfloat16)


def qk_norm_rope_write(qkv, q_weight, k_weight, inv_freq, positions, token_seq, block_table,
                       key_pages, value_pages, *, q_heads, kv_heads, head_dim, rotary_dim, eps,
                       write_kv=True):
    tokens = qkv.shape[0]
    heads = q_heads + (2 * kv_heads if write_kv else 0)
    x = qkv.view(tokens, heads, head_dim).float()

    def norm_rotate(y, w):
        if w is not None:
            y = y * torch.rsqrt(y.square().mean(-1, keepdim=True) + eps) * w
        if rotary_dim:
            half = rotary_dim // 2
            angle = positions.float().view(-1, 1, 1) * inv_freq.view(1, 1, half)
            cos, sin = angle.cos(), angle.sin()
            lo, hi = y[..., :half], y[..., half:rotary_dim]
            y = torch.cat((lo * cos - hi * sin, hi * cos + lo * sin, y[..., rotary_dim:]), dim=-1)
        return y

    q = norm_rotate(x[:, :q_heads], q_weight)
    qkv.view(tokens, heads, head_dim)[:, :q_heads] = q.to(qkv.dtype)
    if not write_kv:
        return
    k = norm_rotate(x[:, q_heads:q_heads + kv_heads], k_weight).to(qkv.dtype)
    v = x[:, q_heads + kv_heads:].to(qkv.dtype)
    block_size = key_pages.shape[2]
    for t in range(tokens):
        pos = int(positions[t])
        page = int(block_table[int(token_seq[t]), pos // block_size])
        assert page >= 0, "token without a page"
        key_pages[page, :, pos % block_size] = k[t]
        value_pages[page, :, :, pos % block_size] = v[t]     # values are stored transposed: [D][slot]


def gather_pages(pages, table_row, length, block_size):
    """[kv_heads, length, D] from pages [blocks, kv_heads, block_size, D]; rows of
    pages that were given back (-1) are NaN so that any read of them shows."""
    kv_heads, head_dim = pages.shape[1], pages.shape[3]
    out = torch.full((kv_heads, length, head_dim), float("nan"))
    for start in range(0, length, block_size):
        page = int(table_row[start // block_size])
        count = min(block_size, length - start)
        if page >= 0:
            out[:, start:start + count] = pages[page, :, :count].float()
    return out


def paged_attention(q, key_pages, value_pages, out, cu_q, ctx_len, block_table, *, num_seqs, max_q_len,
                    q_heads, kv_heads, head_dim, scale, window=None, num_decode=None, max_ctx=None, splits=None):
    block_size = key_pages.shape[2]
    groups = q_heads // kv_heads
    key_pages, value_pages = key_pages.cpu(), value_pages.cpu()
    q_host, table, cu, ctxs = q.float().cpu(), block_table.cpu(), cu_q.cpu(), ctx_len.cpu()
    result = torch.zeros(out.shape, dtype=torch.float32)
    for s in range(num_seqs):
        q0, q1 = int(cu[s]), int(cu[s + 1])
        q_len, ctx = q1 - q0, int(ctxs[s])
        before = ctx - q_len
        keys = gather_pages(key_pages, table[s], ctx, block_size)
        values = gather_pages(value_pages.transpose(2, 3), table[s], ctx, block_size)
        queries = q_host[q0:q1, :q_heads * head_dim].reshape(q_len, q_heads, head_dim)
        for i in range(q_len):
            pos = before + i
            first = 0 if not window else max(0, pos - window + 1)
            for h in range(q_heads):
                kh = h // groups
                scores = (keys[kh, first:pos + 1] @ queries[i, h]) * scale
                probs = torch.softmax(scores, dim=0)
                result[q0 + i, h * head_dim:(h + 1) * head_dim] = probs @ values[kh, first:pos + 1]
    out.copy_(result.to(out.dtype))
    return out


def paged_attention_by_matrices(q, key_pages, value_pages, cu_q, ctx_len, block_table, *, q_heads, kv_heads,
                                head_dim, scale, window=None):
    """``paged_attention`` for long sequences: a whole (sequence, head) at a time as two float32
    matrix products with the causal (and window) mask between them, instead of a token at a time.
    The same formula; ``tests/test_kernel_policies.py`` holds the two against each other.  Returns float32."""
    block_size = key_pages.shape[2]
    groups = q_heads // kv_heads
    result = torch.zeros((q.shape[0], q_heads * head_dim), dtype=torch.float32)
    for s in range(ctx_len.numel()):
        q0, q1 = int(cu_q[s]), int(cu_q[s + 1])
        q_len, ctx = q1 - q0, int(ctx_len[s])
        if q_len == 0:
            continue
        before = ctx - q_len
        keys = gather_pages(key_pages, block_table[s], ctx, block_size)
        values = gather_pages(value_pages.transpose(2, 3), block_table[s], ctx, block_size)
        position = before + torch.arange(q_len).view(-1, 1)
        key_index = torch.arange(ctx).view(1, -1)
        seen = key_index <= position
        if window:
            seen &= key_index > position - window
        keys, values = torch.nan_to_num(keys), torch.nan_to_num(values)   # pages given back lie outside every window
        for h in range(q_heads):
            queries = q[q0:q1, h * head_dim:(h + 1) * head_dim].float()
            scores = (queries @ keys[h // groups].T) * scale
            probs = torch.softmax(scores.masked_fill(~seen, float("-inf")), dim=-1)
            result[q0:q1, h * head_dim:(h + 1) * head_dim] = probs @ values[h // groups]
    return result


def argmax_rows(logits, tokens, status):
    for r in range(logits.shape[0]):
        row = logits[r]
        flags = 0
        if torch.isnan(row).any():
            flags |= 1
        if torch.isposinf(row).any():
            flags |= 2
        if not torch.isfinite(row).any():
            flags |= 4
        status[r] = flags
        tokens[r] = int(torch.argmax(row)) if not flags & 1 else 0


def philox_first_word(counter: int, key: int) -> int:
    """Philox4x32-10 with counter (lo, hi, 0, 0) and key (lo, hi); first word."""
    mask = 0xFFFFFFFF
    c = [counter & mask, (counter >> 32) & mask, 0, 0]
    k = [key & mask, (key >> 32) & mask]
    for _ in range(10):
        p0 = 0xD2511F53 * c[0]
        p1 = 0xCD9E8D57 * c[2]
        c = [((p1 >> 32) ^ c[1] ^ k[0]) & mask, p1 & mask, ((p0 >> 32) ^ c[3] ^ k[1]) & mask, p0 & mask]
        k = [(k[0] + 0x9E3779B9) & mask, (k[1] + 0xBB67AE85) & mask]
    return c[0]


def uniform_from(counter: int, key: int) -> float:
    return (philox_first_word(counter, key) >> 8) / 16777216.0


def kept_after_filters(row, temperature, top_k, top_p, min_p):
    """(weights, kept) of one row in float64 after temperature, top-k, top-p, min-p in the order and
    with the rules of the reference (src/forge_engine/sampling.py:83-140): e_i = exp((x_i - max) / T);
    top-k keeps the k largest; top-p keeps a token if the probability of all larger ones, within what
    top-k left, is <= top_p; min-p keeps e_i >= min_p (the largest e is 1)."""
    # the logit as the kernel forms it, in float32: (max - x) * (1 / T); everything after it in float64
    y = (row.float().max() - row.float()) * torch.tensor(1.0, dtype=torch.float32).div(temperature)
    x = -y.double()
    e = torch.exp(x)
    kept = torch.ones_like(e, dtype=torch.bool)
    if top_k and top_k < len(row):
        kth = torch.topk(x, top_k).values[-1]
        kept &= x >= kth
    if top_p < 1.0:
        masked = torch.where(kept, e, torch.zeros_like(e))
        order = torch.argsort(x, descending=True, stable=True)
        before = masked[order].cumsum(0) - masked[order]
        keep_sorted = before <= top_p * masked.sum()
        by_p = torch.zeros_like(kept)
        by_p[order] = keep_sorted
        kept &= by_p
    if min_p > 0.0:
        kept &= e >= min_p
    return e, kept


def unpack_sample_params(params):
    """Rows of (temperature, top_k, top_p, min_p, seed, draw index) from the packed int32 words."""
    words = params.cpu().contiguous()
    floats = words.view(torch.float32)
    rows = []
    for r in range(words.shape[0]):
        low = [int(v) & 0xFFFFFFFF for v in words[r, 4:8]]
        rows.append((float(floats[r, 0]), int(words[r, 1]), float(floats[r, 2]), float(floats[r, 3]),
                     low[0] | (low[1] << 32), low[2] | (low[3] << 32)))
    return rows


def sample_filtered_rows(logits, params, tokens, status, any_top_k=True, any_top_p=True):
    """Arg-max (temperature 0), or the filters above and an inverse CDF in float64 over what they
    kept, in token order, with the same uniform as the kernel; the kernel's sums of 2^-40 steps may
    pick a neighbour when the target falls within rounding of a boundary (tests allow for that)."""
    for r, (temperature, top_k, top_p, min_p, seed, draw) in enumerate(unpack_sample_params(params)):
        row = logits[r]
        flags = 0
        if torch.isnan(row).any():
            flags |= 1
        if torch.isposinf(row).any():
            flags |= 2
        if not torch.isfinite(row).any():
            flags |= 4
        status[r] = flags
        if flags:
            tokens[r] = 0
            continue
        if not temperature > 0:
            tokens[r] = int(torch.argmax(row))
            continue
        e, kept = kept_after_filters(row, temperature, top_k, top_p, min_p)
        cdf = torch.where(kept, e, torch.zeros_like(e)).cumsum(0)
        target = uniform_from(draw, seed) * float(cdf[-1])
        pick = int(torch.searchsorted(cdf, torch.tensor(target, dtype=torch.float64), right=True))
        tokens[r] = min(pick, logits.shape[1] - 1)


def decode_prepare_supported(*args, **kwargs):
    return False        # on the CPU a step of single tokens takes the two references below in turn


def linear_in_parts(x, weight):
    return None


# Key splits of the bfloat16 decode attention that the GPU tests launch (every count the kernel takes:
# 1 to 4, 5 to 8 and 9 to 16 merge with all loads in one round, 17 to 64 in a loop)
DECODE_SPLITS_TESTED = tuple(range(1, 65))


NAMES = ("decode_prepare_supported", "linear_in_parts", "embed_rows", "add_rmsnorm", "add_rows", "swiglu", "gemm_nt_f32", "linear", "linear_update", "linear_swiglu", "gemm_skinny",
         "qk_norm_rope_write", "paged_attention", "argmax_rows", "sample_filtered_rows")


def install(monkeypatch):
    """Patch the references in for the HIP kernels (CPU tests only)."""
    from forge_engine_amd.kernels import ops

    for name in NAMES:
        monkeypatch.setattr(ops, name, globals()[name])
