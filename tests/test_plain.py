"""Pins for the plain implementation: vectors held by the reference's own tests,
special cases that reduce to a library routine, and invariants.  Each is chosen
so that a plausible mistake (wrong sign or pairing, a norm in the wrong place)
fails it."""

from __future__ import annotations

import math

import pytest
import torch
import torch.nn.functional as F

import plain_qwen3 as plain
from conftest import TINY


def test_rms_norm_reference_vector():
    # tests/test_qwen3.py:34-44 of the reference
    x = torch.tensor([[1.0, -2.0, 3.0, -4.0]])
    w = torch.tensor([1.0, 2.0, 3.0, 4.0])
    expected = x * torch.rsqrt(x.square().mean(dim=-1, keepdim=True) + 1e-6) * w
    torch.testing.assert_close(plain.rms_norm(x, w, 1e-6), expected)
    # hand value: mean square 7.5
    assert plain.rms_norm(x, w, 1e-6)[0, 3].item() == pytest.approx(-16 / math.sqrt(7.5), rel=1e-6)


def test_rms_norm_is_library_rms_norm():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(5, 24, generator=g)
    w = torch.randn(24, generator=g)
    torch.testing.assert_close(plain.rms_norm(x, w, 1e-5), F.rms_norm(x, (24,), w, 1e-5))


def test_add_rms_norm_reference_vector():
    # tests/test_kernels.py:20-36 of the reference
    r = torch.tensor([[1.0, -2.0, 3.0, -4.0]])
    u = torch.tensor([[0.5, 1.0, -1.5, 2.0]])
    w = torch.tensor([1.0, 2.0, 3.0, 4.0])
    summed, normed = plain.add_rms_norm(r, u, w, 1e-6)
    s = r + u
    torch.testing.assert_close(summed, s)
    torch.testing.assert_close(normed, s * torch.rsqrt(s.square().mean(-1, keepdim=True) + 1e-6) * w)
    zero_sum, zero_norm = plain.add_rms_norm(r, torch.zeros_like(r), w, 1e-6)
    torch.testing.assert_close(zero_norm, plain.rms_norm(r, w, 1e-6))


def test_rotary_sign_and_pairing():
    # D = 4, theta = 10000: inv_freq = [1, 0.01].  A unit vector in dim 0 at
    # position 1 turns into (cos 1, 0, sin 1, 0): partner of dim j is j + D/2,
    # and the second half gets +sin.
    cos, sin = plain.rotary_tables(torch.tensor([1]), 4, 10000.0)
    x = torch.tensor([[[1.0, 0.0, 0.0, 0.0]]])
    out = plain.apply_rotary(x, cos, sin)[0, 0]
    torch.testing.assert_close(out, torch.tensor([math.cos(1.0), 0.0, math.sin(1.0), 0.0]))
    y = torch.tensor([[[0.0, 1.0, 0.0, 0.0]]])
    out = plain.apply_rotary(y, cos, sin)[0, 0]
    torch.testing.assert_close(out, torch.tensor([0.0, math.cos(0.01), 0.0, math.sin(0.01)]))


def test_rotary_position_zero_is_identity_and_norm_kept():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(3, 6, 16, generator=g)
    cos, sin = plain.rotary_tables(torch.arange(6), 16, 1e6)
    out = plain.apply_rotary(x, cos, sin)
    torch.testing.assert_close(out[:, 0], x[:, 0])
    pair_norm_in = x[..., :8] ** 2 + x[..., 8:] ** 2
    pair_norm_out = out[..., :8] ** 2 + out[..., 8:] ** 2
    torch.testing.assert_close(pair_norm_out, pair_norm_in)


def test_rotary_scores_depend_on_distance_only():
    g = torch.Generator().manual_seed(3)
    q = torch.randn(1, 1, 32, generator=g).double()
    k = torch.randn(1, 1, 32, generator=g).double()

    def score(pq, pk):
        cq, sq = plain.rotary_tables(torch.tensor([pq]), 32, 10000.0)
        ck, sk = plain.rotary_tables(torch.tensor([pk]), 32, 10000.0)
        return (plain.apply_rotary(q, cq.double(), sq.double())
                * plain.apply_rotary(k, ck.double(), sk.double())).sum().item()

    assert score(9, 4) == pytest.approx(score(25, 20), abs=1e-5)
    assert abs(score(9, 4) - score(9, 5)) > 1e-3


def test_attention_is_library_attention_after_group_expansion():
    # tests/test_kernels.py:91-105 of the reference uses the same library call
    g = torch.Generator().manual_seed(7)
    q = torch.randn(6, 9, 8, generator=g)
    k = torch.randn(2, 9, 8, generator=g)
    v = torch.randn(2, 9, 8, generator=g)
    got = plain.causal_attention(q, k, v, 8**-0.5)
    want = F.scaled_dot_product_attention(
        q.unsqueeze(0), k.repeat_interleave(3, 0).unsqueeze(0),
        v.repeat_interleave(3, 0).unsqueeze(0), is_causal=True)[0]
    torch.testing.assert_close(got, want, atol=1e-6, rtol=1e-6)


def test_attention_group_mapping_is_blockwise():
    # query heads 0,1 read kv head 0 and heads 2,3 read kv head 1 (h // G), not h % Hkv
    q = torch.zeros(4, 1, 4)
    k = torch.zeros(2, 1, 4)
    v = torch.stack((torch.full((1, 4), 1.0), torch.full((1, 4), 2.0)))
    out = plain.causal_attention(q, k, v, 0.5)
    assert out[:, 0, 0].tolist() == [1.0, 1.0, 2.0, 2.0]


def test_attention_window_keeps_last_w_keys():
    g = torch.Generator().manual_seed(8)
    q = torch.randn(1, 7, 4, generator=g)
    k = torch.randn(1, 7, 4, generator=g)
    v = torch.randn(1, 7, 4, generator=g)
    got = plain.causal_attention(q, k, v, 0.5, window=3)[0, 6]
    s = (k[0, 4:7] @ q[0, 6]) * 0.5
    want = torch.softmax(s, 0) @ v[0, 4:7]
    torch.testing.assert_close(got, want)


def test_swiglu_is_library_expression():
    # tests/test_cute_swiglu.py:18-27 of the reference: seed 23, [3,8] x [12,8]
    torch.manual_seed(23)
    x = torch.randn(3, 8)
    wg = torch.randn(12, 8)
    wu = torch.randn(12, 8)
    wd = torch.eye(12)
    weights = {"m.gate_proj.weight": wg, "m.up_proj.weight": wu, "m.down_proj.weight": wd}
    torch.testing.assert_close(plain.swiglu_mlp(x, weights, "m"), F.silu(x @ wg.T) * (x @ wu.T))


@pytest.mark.parametrize("name", ["A", "B"])
def test_shift_of_all_positions_changes_nothing(name):
    config = TINY[name]
    w = plain.random_weights(config, 5)
    ids = torch.randint(0, config["vocab_size"], (12,), generator=torch.Generator().manual_seed(0))
    a = plain.forward(w, config, ids)
    b = plain.forward(w, config, ids, first_position=37)
    torch.testing.assert_close(a, b, atol=2e-5, rtol=1e-4)
    shuffled = plain.forward(w, config, ids.flip(0))
    assert (a - shuffled.flip(0)).abs().max() > 1e-3   # positions do matter


@pytest.mark.parametrize("name", ["A", "B"])
def test_prefix_logits_do_not_see_later_tokens(name):
    config = TINY[name]
    w = plain.random_weights(config, 6)
    ids = torch.randint(0, config["vocab_size"], (10,), generator=torch.Generator().manual_seed(1))
    full = plain.forward(w, config, ids)
    torch.testing.assert_close(full[:6], plain.forward(w, config, ids[:6]), atol=1e-6, rtol=1e-5)


def test_query_scale_is_removed_by_the_per_head_norm():
    # q_norm sits between the projection and the rotation: scaling W_q leaves
    # the logits unchanged (up to eps); without the norm they would change.
    config = TINY["A"]
    w = plain.random_weights(config, 9)
    ids = [3, 200, 17, 17, 64]
    a = plain.forward(w, config, ids)
    w2 = dict(w)
    for i in range(config["num_hidden_layers"]):
        name = f"model.layers.{i}.self_attn.q_proj.weight"
        w2[name] = w[name] * 8.0
    torch.testing.assert_close(plain.forward(w2, config, ids), a, atol=1e-5, rtol=1e-4)


def test_zeroed_output_projections_reduce_to_norm_and_head():
    config = TINY["B"]
    w = plain.random_weights(config, 10)
    for i in range(config["num_hidden_layers"]):
        w[f"model.layers.{i}.self_attn.o_proj.weight"].zero_()
        w[f"model.layers.{i}.mlp.down_proj.weight"].zero_()
    ids = torch.tensor([5, 6, 7])
    e = w["model.embed_tokens.weight"][ids]
    want = F.rms_norm(e, (config["hidden_size"],), w["model.norm.weight"], config["rms_norm_eps"]) @ w["lm_head.weight"].T
    torch.testing.assert_close(plain.forward(w, config, ids), want, atol=1e-6, rtol=1e-5)


def test_feed_forward_reads_the_normalised_sum():
    # one layer, attention silenced: h = e + mlp(norm_post(e))
    config = dict(TINY["A"], num_hidden_layers=1)
    w = plain.random_weights(config, 11)
    w["model.layers.0.self_attn.o_proj.weight"].zero_()
    ids = torch.tensor([9, 8])
    e = w["model.embed_tokens.weight"][ids]
    y = F.rms_norm(e, (64,), w["model.layers.0.post_attention_layernorm.weight"], 1e-6)
    m = (F.silu(y @ w["model.layers.0.mlp.gate_proj.weight"].T) * (y @ w["model.layers.0.mlp.up_proj.weight"].T)) @ w["model.layers.0.mlp.down_proj.weight"].T
    z = F.rms_norm(e + m, (64,), w["model.norm.weight"], 1e-6)
    torch.testing.assert_close(plain.forward(w, config, ids), z @ w["model.embed_tokens.weight"].T, atol=1e-6, rtol=1e-5)


def test_sampling_filter_vectors():
    # tests/test_sampling.py:47-81 of the reference
    def kept(x):
        return torch.isfinite(x).nonzero()[:, 1].tolist()

    assert kept(plain.filter_logits(torch.tensor([[0.0, 3.0, 2.0, 1.0]]), 1.0, top_k=2)) == [1, 2]
    assert kept(plain.filter_logits(torch.tensor([[5.0, 4.0, 0.0]]), 1.0, top_p=0.7)) == [0]
    assert kept(plain.filter_logits(torch.tensor([[0.0, -1.0, -3.0]]), 1.0, min_p=0.2)) == [0, 1]


def test_key_scale_is_removed_by_the_per_head_norm():
    # k_norm sits between the k projection and the rotation (qwen3.py:146-150): scaling W_k
    # leaves the logits unchanged (up to eps, which is why the configuration with the smaller
    # eps is used); without k_norm every score would scale.
    config = TINY["A"]
    w = plain.random_weights(config, 12)
    ids = [3, 200, 17, 17, 64, 9]
    a = plain.forward(w, config, ids)
    w2 = dict(w)
    for i in range(config["num_hidden_layers"]):
        name = f"model.layers.{i}.self_attn.k_proj.weight"
        w2[name] = w[name] * 8.0
    torch.testing.assert_close(plain.forward(w2, config, ids), a, atol=1e-5, rtol=1e-4)
    # the control: the same scaling of W_v does change them (nothing normalises v)
    w3 = dict(w)
    for i in range(config["num_hidden_layers"]):
        name = f"model.layers.{i}.self_attn.v_proj.weight"
        w3[name] = w[name] * 8.0
    assert (plain.forward(w3, config, ids) - a).abs().max() > 1e-3


def test_values_are_not_normalised():
    # v goes from its projection straight into the weighted sum (qwen3.py:151-155): with the
    # feed-forward silenced, scaling W_v by c scales the layer's update of the stream by c.
    config = dict(TINY["A"], num_hidden_layers=1)
    w = plain.random_weights(config, 13)
    w["model.layers.0.mlp.down_proj.weight"].zero_()
    ids = torch.tensor([9, 8, 100, 7])
    e = w["model.embed_tokens.weight"][ids]
    _, hidden = plain.forward(w, config, ids, return_hidden=True)
    update = hidden[0] - e
    w2 = dict(w)
    w2["model.layers.0.self_attn.v_proj.weight"] = w["model.layers.0.self_attn.v_proj.weight"] * 3.0
    _, hidden2 = plain.forward(w2, config, ids, return_hidden=True)
    assert update.abs().max() > 1e-4
    torch.testing.assert_close(hidden2[0] - e, 3.0 * update, atol=1e-6, rtol=1e-5)


def _hand_attention_weights(a: float, b: float) -> dict:
    eye = torch.eye(4)
    return {"p.q_proj.weight": eye.clone(), "p.k_proj.weight": eye.clone(), "p.v_proj.weight": eye.clone(),
            "p.o_proj.weight": eye.clone(), "p.q_norm.weight": torch.full((4,), a),
            "p.k_norm.weight": torch.full((4,), b)}


def test_attention_block_by_hand_scale_norms_and_values():
    # One head of size 4, identity projections, theta so large that dims 1 and 3 do not turn
    # (dims 0 and 2 hold zeros).  Rows (0,3,0,4) and (0,4,0,-3) have RMS 2.5, so after the
    # per-head norms q = a x / 2.5 and k = b x / 2.5: for the second token q1.k0 = 0 and
    # q1.k1 = 4ab, and its scores are (0, 4ab * D^-0.5) = (0, 2ab)  (qwen3.py:129,189-190).
    # The values are the rows themselves.  Scale 1.0, a missing k_norm or a normalised v
    # each give another result.
    a, b = 1.5, 0.5
    config = {"num_attention_heads": 1, "num_key_value_heads": 1, "head_dim": 4, "rms_norm_eps": 1e-12,
              "rope_theta": 1e30}
    x = torch.tensor([[0.0, 3.0, 0.0, 4.0], [0.0, 4.0, 0.0, -3.0]])
    out = plain.attention_block(x, _hand_attention_weights(a, b), "p", config, torch.arange(2))
    p1 = math.exp(2 * a * b) / (1.0 + math.exp(2 * a * b))
    torch.testing.assert_close(out[0], x[0])
    torch.testing.assert_close(out[1], (1 - p1) * x[0] + p1 * x[1], atol=1e-6, rtol=1e-6)


def test_attention_block_is_library_attention_with_its_default_scale():
    # norms and rotation by hand, then the library's attention, whose default scale is
    # 1/sqrt(head size): pins the block's own choice of scale, that both q and k are
    # normalised and that v is not.
    config = dict(TINY["B"])
    heads, kv_heads, d = config["num_attention_heads"], config["num_key_value_heads"], config["head_dim"]
    w = plain.random_weights(config, 14)
    prefix = "model.layers.1.self_attn"
    g = torch.Generator().manual_seed(15)
    x = torch.randn(7, config["hidden_size"], generator=g)
    q = (x @ w[f"{prefix}.q_proj.weight"].T).view(7, heads, d)
    k = (x @ w[f"{prefix}.k_proj.weight"].T).view(7, kv_heads, d)
    v = (x @ w[f"{prefix}.v_proj.weight"].T).view(7, kv_heads, d)
    q = F.rms_norm(q, (d,), w[f"{prefix}.q_norm.weight"], config["rms_norm_eps"]).transpose(0, 1)
    k = F.rms_norm(k, (d,), w[f"{prefix}.k_norm.weight"], config["rms_norm_eps"]).transpose(0, 1)
    cos, sin = plain.rotary_tables(torch.arange(7), d, config["rope_theta"])
    q, k = plain.apply_rotary(q, cos, sin), plain.apply_rotary(k, cos, sin)
    groups = heads // kv_heads
    want = F.scaled_dot_product_attention(
        q.unsqueeze(0), k.repeat_interleave(groups, 0).unsqueeze(0),
        v.transpose(0, 1).repeat_interleave(groups, 0).unsqueeze(0), is_causal=True)[0]
    want = want.transpose(0, 1).reshape(7, heads * d) @ w[f"{prefix}.o_proj.weight"].T
    got = plain.attention_block(x, w, prefix, config, torch.arange(7))
    torch.testing.assert_close(got, want, atol=1e-6, rtol=1e-5)


def _one_layer_attention_only(seed: int, **overrides):
    """A one-layer model of configuration A whose feed-forward is silenced: the layer's update of
    the stream is the attention block's output alone."""
    config = dict(TINY["A"], num_hidden_layers=1, **overrides)
    w = plain.random_weights(config, seed)
    w["model.layers.0.mlp.down_proj.weight"].zero_()
    return config, w


def test_input_norm_weight_scales_what_the_projections_read():
    # x = w_in * normalised(h) feeds q, k and v (qwen3.py:248-253): zeroing element j of the input
    # norm's weight is zeroing column j of W_q, W_k and W_v; a unit weight, or the post-attention
    # norm's weight in its place, breaks the first equality.  Scaling the weight by c scales v by c
    # and leaves q and k to their own norms: the update scales by c (the eps is made tiny for that).
    config, w = _one_layer_attention_only(21, rms_norm_eps=1e-12)
    p = "model.layers.0"
    ids = torch.tensor([9, 8, 100, 7, 33])
    e = w["model.embed_tokens.weight"][ids]
    _, hidden = plain.forward(w, config, ids, return_hidden=True)
    update = hidden[0] - e
    assert update.abs().max() > 1e-4
    for j in (0, 17, 63):
        gated = dict(w)
        gated[f"{p}.input_layernorm.weight"] = w[f"{p}.input_layernorm.weight"].clone()
        gated[f"{p}.input_layernorm.weight"][j] = 0.0
        cut = dict(w)
        for name in ("q_proj", "k_proj", "v_proj"):
            cut[f"{p}.self_attn.{name}.weight"] = w[f"{p}.self_attn.{name}.weight"].clone()
            cut[f"{p}.self_attn.{name}.weight"][:, j] = 0.0
        _, a = plain.forward(gated, config, ids, return_hidden=True)
        _, b = plain.forward(cut, config, ids, return_hidden=True)
        torch.testing.assert_close(a[0], b[0], atol=1e-7, rtol=1e-5)
        assert (a[0] - hidden[0]).abs().max() > 1e-5             # and element j did matter
    scaled = dict(w)
    scaled[f"{p}.input_layernorm.weight"] = w[f"{p}.input_layernorm.weight"] * 3.0
    _, c = plain.forward(scaled, config, ids, return_hidden=True)
    torch.testing.assert_close(c[0] - e, 3.0 * update, atol=1e-7, rtol=1e-4)
    # the post-attention norm's weight does not reach the attention at all (the feed-forward is silent)
    other = dict(w)
    other[f"{p}.post_attention_layernorm.weight"] = w[f"{p}.post_attention_layernorm.weight"] * 5.0
    _, d = plain.forward(other, config, ids, return_hidden=True)
    torch.testing.assert_close(d[0], hidden[0], atol=0, rtol=0)


def test_input_norm_uses_the_configurations_eps():
    # One token: its attention output is its own value whatever q and k are, so the layer's update
    # is W_o expand(W_v x) with x = w_in * e / sqrt(mean(e^2) + eps) (qwen3.py:99-105,237,248).
    # The embedding row is scaled so that mean(e^2) equals eps exactly: the norm then divides by
    # sqrt(2) times the row's RMS, a factor that another eps (1e-6, say) would not give.
    eps = 1e-3
    config, w = _one_layer_attention_only(22, rms_norm_eps=eps)
    p = "model.layers.0"
    token = 41
    row = w["model.embed_tokens.weight"][token]
    row *= math.sqrt(eps) / row.square().mean().sqrt()
    e = w["model.embed_tokens.weight"][token]
    assert abs(float(e.square().mean()) - eps) < 1e-9
    x = w[f"{p}.input_layernorm.weight"] * e / (math.sqrt(2.0) * e.square().mean().sqrt())
    groups = config["num_attention_heads"] // config["num_key_value_heads"]
    v = (w[f"{p}.self_attn.v_proj.weight"] @ x).view(config["num_key_value_heads"], config["head_dim"])
    want = w[f"{p}.self_attn.o_proj.weight"] @ v.repeat_interleave(groups, dim=0).reshape(-1)
    _, hidden = plain.forward(w, config, [token], return_hidden=True)
    torch.testing.assert_close(hidden[0][0] - e, want, atol=1e-8, rtol=1e-5)
    wrong = w[f"{p}.self_attn.o_proj.weight"] @ (v * math.sqrt(2.0)).repeat_interleave(groups, dim=0).reshape(-1)   # what eps -> 0 gives
    assert (hidden[0][0] - e - wrong).abs().max() > 1e-4 * wrong.abs().max()


@pytest.mark.parametrize("name", ["A", "B"])
def test_layers_run_in_the_order_of_their_numbers(name):
    # the stream after layer i of an L-layer model is the output of the (i + 1)-layer model made
    # of the first i + 1 layers' tensors alone (qwen3.py:328-331)
    config = TINY[name]
    w = plain.random_weights(config, 23)
    ids = torch.randint(0, config["vocab_size"], (9,), generator=torch.Generator().manual_seed(2))
    _, hidden = plain.forward(w, config, ids, return_hidden=True)
    assert len(hidden) == config["num_hidden_layers"]
    for count in range(1, config["num_hidden_layers"]):
        shorter = dict(config, num_hidden_layers=count)
        first = {k: v for k, v in w.items() if not k.startswith("model.layers.")
                 or int(k.split(".")[2]) < count}
        _, partial = plain.forward(first, shorter, ids, return_hidden=True)
        torch.testing.assert_close(hidden[count - 1], partial[-1], atol=0, rtol=0)
        assert (hidden[count - 1] - hidden[count]).abs().max() > 1e-4


def test_attention_biases_are_added_to_the_projections_before_the_head_norms():
    # attention_bias (qwen3.py:115-122): with W_q = W_k = 0 every query is norm(b_q) and every key
    # norm(b_k), each turned by its position; v = W_v x + b_v; the output gets b_o.  The biases'
    # RMS is far from one, so a bias added after the per-head norm, like a bias that is dropped,
    # gives other scores; values differ from token to token, so the scores matter.
    config = dict(TINY["B"], attention_bias=True)
    heads, kv_heads, d = config["num_attention_heads"], config["num_key_value_heads"], config["head_dim"]
    w = plain.random_weights(config, 24)
    prefix = "model.layers.0.self_attn"
    g = torch.Generator().manual_seed(25)
    w[f"{prefix}.q_proj.weight"].zero_()
    w[f"{prefix}.k_proj.weight"].zero_()
    w[f"{prefix}.v_proj.weight"] *= 20.0
    biases = {"q_proj": torch.randn(heads * d, generator=g) * 3.0, "k_proj": torch.randn(kv_heads * d, generator=g) * 3.0,
              "v_proj": torch.randn(kv_heads * d, generator=g), "o_proj": torch.randn(config["hidden_size"], generator=g)}
    for name, bias in biases.items():
        w[f"{prefix}.{name}.bias"] = bias
    length = 6
    x = torch.randn(length, config["hidden_size"], generator=g)
    eps = config["rms_norm_eps"]
    q = F.rms_norm(biases["q_proj"].view(heads, d), (d,), w[f"{prefix}.q_norm.weight"], eps)
    k = F.rms_norm(biases["k_proj"].view(kv_heads, d), (d,), w[f"{prefix}.k_norm.weight"], eps)
    q = q.unsqueeze(1).expand(heads, length, d)
    k = k.unsqueeze(1).expand(kv_heads, length, d)
    v = (x @ w[f"{prefix}.v_proj.weight"].T + biases["v_proj"]).view(length, kv_heads, d).transpose(0, 1)
    cos, sin = plain.rotary_tables(torch.arange(length), d, config["rope_theta"])
    q, k = plain.apply_rotary(q, cos, sin), plain.apply_rotary(k, cos, sin)
    groups = heads // kv_heads
    want = F.scaled_dot_product_attention(q.unsqueeze(0), k.repeat_interleave(groups, 0).unsqueeze(0),
                                          v.repeat_interleave(groups, 0).unsqueeze(0), is_causal=True)[0]
    want = want.transpose(0, 1).reshape(length, heads * d) @ w[f"{prefix}.o_proj.weight"].T + biases["o_proj"]
    got = plain.attention_block(x, w, prefix, config, torch.arange(length))
    torch.testing.assert_close(got, want, atol=1e-5, rtol=1e-5)
    # each of the four biases matters here
    for name in biases:
        without = {key: value for key, value in w.items() if key != f"{prefix}.{name}.bias"}
        assert (plain.attention_block(x, without, prefix, config, torch.arange(length)) - want).abs().max() > 1e-3, name
    # and a bias added after the norm would give other scores: the unnormalised biases are three times as long
    unnormalised = plain.apply_rotary(biases["q_proj"].view(heads, d).unsqueeze(1).expand(heads, length, d), cos, sin)
    other = F.scaled_dot_product_attention(unnormalised.unsqueeze(0), k.repeat_interleave(groups, 0).unsqueeze(0),
                                           v.repeat_interleave(groups, 0).unsqueeze(0), is_causal=True)[0]
    other = other.transpose(0, 1).reshape(length, heads * d) @ w[f"{prefix}.o_proj.weight"].T + biases["o_proj"]
    assert (other - want).abs().max() > 1e-3
