"""What pins the plain implementation beside the reference's text: vectors the reference's own
tests and fixtures hold, special cases that reduce to a library routine, and invariants, each
chosen so that a plausible mistake (a wrong sign or pairing in the rotation, heads grouped in
the wrong order, a mask off by one, a norm with 1 + w) fails it."""
import math
import os

import pytest
import torch
import torch.nn.functional as F

import plain_llama as plain
from conftest import TINY_A, TINY_B

LLAMA32 = dict(head_dim=64, theta=500000.0, scaling={
    "rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
    "original_max_position_embeddings": 8192})

# crates/model/src/rope.rs:146-156, printed there from transformers for the Llama 3.2 1B config.
LLAMA32_INV_FREQ = [
    1.000000000e+00, 6.636012793e-01, 4.403666258e-01, 2.922278345e-01,
    1.939227581e-01, 1.286873817e-01, 8.539710194e-02, 5.666961893e-02,
    3.760603070e-02, 2.495540865e-02, 1.656044088e-02, 1.098952908e-02,
    7.292665076e-03, 4.839421250e-03, 3.211446106e-03, 1.290548011e-03,
    4.295567051e-04, 9.708286234e-05, 1.946163866e-05, 1.291476747e-05,
    8.570255886e-06, 5.687232260e-06, 3.774054449e-06, 2.504467147e-06,
    1.661967417e-06, 1.102883630e-06, 7.318749340e-07, 4.856731266e-07,
    3.222932889e-07, 2.138742303e-07, 1.419272024e-07, 9.418306490e-08,
]


def product_inv_freqs(head_dim, theta, scaling):
    from rust_llm_inference_server_amd.parts.rope import inverse_frequencies
    return inverse_frequencies(head_dim, theta, scaling)


@pytest.mark.parametrize("fn", [plain.inv_freqs, product_inv_freqs])
def test_inv_freq_matches_the_reference_vector(fn):
    got = fn(LLAMA32["head_dim"], LLAMA32["theta"], LLAMA32["scaling"])
    want = torch.tensor(LLAMA32_INV_FREQ)
    assert got.dtype == torch.float32 and got.shape == (32,)
    assert ((got - want) / want).abs().max().item() < 1e-6          # rope.rs:138-141


@pytest.mark.parametrize("fn", [plain.inv_freqs, product_inv_freqs])
def test_inv_freq_matches_the_reference_fixture(fn):
    """The parity fixture the reference ships holds the same vector as a tensor
    (scripts/parity/dump_reference.py:116-119); read with the safetensors package."""
    root = os.environ.get("RLIS_REFERENCE_DIR", "/root/reference")
    path = os.path.join(root, "tests/fixtures/parity/reference.safetensors")
    if not os.path.exists(path):
        pytest.skip(f"the reference's fixture is not at {path} (set RLIS_REFERENCE_DIR to the "
                    "reference checkout); the same 32 values are pinned from rope.rs:146-156 above")
    from safetensors import safe_open
    with safe_open(path, framework="pt") as f:
        want = f.get_tensor("inv_freq")
    got = fn(LLAMA32["head_dim"], LLAMA32["theta"], LLAMA32["scaling"])
    assert ((got - want) / want).abs().max().item() < 1e-6


@pytest.mark.parametrize("fn", [plain.inv_freqs, product_inv_freqs])
def test_llama3_bands(fn):
    """Tiny B (theta 5e5, d 32, factor 8, low 1, high 4, original 64): wavelengths 6.28, 14.3,
    32.4, 73.6, ...: two frequencies are kept, one is blended, the rest are divided by 8; and
    without scaling the frequencies are theta^(-2j/d)."""
    sc = TINY_B["rope_scaling"]
    base = fn(32, 500000.0, None)
    torch.testing.assert_close(base, 500000.0 ** (-torch.arange(0, 32, 2) / 32), rtol=1e-6, atol=0)
    got = fn(32, 500000.0, sc)
    ratio = got / base
    assert torch.equal(ratio[:2], torch.ones(2))
    assert 1 / 8 < ratio[2].item() < 1
    torch.testing.assert_close(ratio[3:], torch.full((13,), 1 / 8), rtol=1e-6, atol=0)
    assert (got[1:] < got[:-1]).all()
    assert torch.equal(fn(32, 500000.0, sc), plain.inv_freqs(32, 500000.0, sc))


def test_rms_norm_reduces_to_the_library_routine():
    x, w = torch.randn(5, 100) * 3, 1 + 0.1 * torch.randn(100)
    for eps in (1e-5, 1e-6, 0.3):
        torch.testing.assert_close(plain.rms_norm(x, w, eps), F.rms_norm(x, (100,), w, eps),
                                   rtol=1e-6, atol=1e-6)
    y = plain.rms_norm(x, torch.ones(100), 0.0)
    torch.testing.assert_close((y * y).mean(-1), torch.ones(5), rtol=1e-5, atol=1e-5)
    # the weight multiplies directly: a zero weight gives zero (1 + w would give the norm)
    assert plain.rms_norm(x, torch.zeros(100), 1e-5).abs().max().item() == 0.0


def test_linear_and_swiglu_reduce_to_library_routines():
    x, w = torch.randn(4, 10), torch.randn(7, 10)
    torch.testing.assert_close(plain.linear(x, w), F.linear(x, w))
    ws = {"m.gate_proj.weight": torch.randn(12, 10), "m.up_proj.weight": torch.randn(12, 10),
          "m.down_proj.weight": torch.randn(10, 12)}
    want = F.linear(F.silu(F.linear(x, ws["m.gate_proj.weight"])) * F.linear(x, ws["m.up_proj.weight"]),
                    ws["m.down_proj.weight"])
    torch.testing.assert_close(plain.swiglu_mlp(x, ws, "m"), want, rtol=1e-5, atol=1e-5)


def test_rope_pairs_halves_with_the_right_sign():
    """d = 4, inverse frequencies (1, f): the unit vector e0 at position p becomes
    (cos p, 0, sin p, 0): dim 0 pairs with dim 2 (not dim 1), and the rotation is
    counter-clockwise (rope.rs:5-8: o_j = x_j cos - x_{j+d/2} sin)."""
    inv = torch.tensor([1.0, 0.25])
    p = 3
    cos, sin = plain.rope_tables(inv, [p])
    x = torch.tensor([[[1.0, 0.0, 0.0, 0.0]]])
    got = plain.rope_apply(x, cos, sin)[0, 0]
    torch.testing.assert_close(got, torch.tensor([math.cos(p), 0.0, math.sin(p), 0.0]))
    y = torch.tensor([[[0.0, 1.0, 0.0, 0.0]]])
    got = plain.rope_apply(y, cos, sin)[0, 0]
    torch.testing.assert_close(got, torch.tensor([0.0, math.cos(0.25 * p), 0.0, math.sin(0.25 * p)]))


def test_rope_invariants():
    inv = plain.inv_freqs(32, 10000.0, None)
    q, k = torch.randn(2, 1, 32), torch.randn(2, 1, 32)
    cos0, sin0 = plain.rope_tables(inv, [0])
    torch.testing.assert_close(plain.rope_apply(q, cos0, sin0), q)              # position 0
    c, s = plain.rope_tables(inv, [17])
    torch.testing.assert_close(plain.rope_apply(q, c, s).norm(dim=-1), q.norm(dim=-1),
                               rtol=1e-5, atol=1e-5)                             # norm kept

    def dot(m, n):
        cm, sm = plain.rope_tables(inv, [m])
        cn, sn = plain.rope_tables(inv, [n])
        return (plain.rope_apply(q, cm, sm) * plain.rope_apply(k, cn, sn)).sum(-1)

    torch.testing.assert_close(dot(5, 2), dot(45, 42), rtol=1e-4, atol=1e-4)     # only m - n counts
    assert (dot(5, 2) - dot(5, 3)).abs().max().item() > 1e-3


def test_causal_mask_vectors():
    m = plain.causal_mask(2, 1)                       # attention.rs:299-305
    assert m.tolist() == [[0.0, 0.0, float("-inf")], [0.0, 0.0, 0.0]]
    w = plain.causal_mask(3, 2, window=2)
    inf = float("-inf")
    assert w.tolist() == [[inf, 0.0, 0.0, inf, inf], [inf, inf, 0.0, 0.0, inf],
                          [inf, inf, inf, 0.0, 0.0]]


def repeat_kv(x, n_rep):                              # attention.rs:240-245
    nkv, t, d = x.shape
    return x.unsqueeze(1).expand(nkv, n_rep, t, d).reshape(nkv * n_rep, t, d)


def test_repeat_kv_maps_heads_in_groups():
    x = torch.arange(4.0).reshape(2, 2, 1)
    assert repeat_kv(x, 3).flatten().tolist() == [0, 1, 0, 1, 0, 1, 2, 3, 2, 3, 2, 3]


def test_grouped_attention_matches_the_textbook_and_the_library():
    nh, nkv, seq, start, d = 8, 2, 5, 3, 16            # attention.rs:259-272
    q, k, v = torch.randn(nh, seq, d), torch.randn(nkv, start + seq, d), torch.randn(nkv, start + seq, d)
    mask = plain.causal_mask(seq, start)
    got = plain.gqa_attention(q, k, v, mask)
    kr, vr = repeat_kv(k, nh // nkv), repeat_kv(v, nh // nkv)
    s = q @ kr.transpose(1, 2) / math.sqrt(d) + mask
    torch.testing.assert_close(got, torch.softmax(s, -1) @ vr, rtol=1e-5, atol=1e-5)
    lib = F.scaled_dot_product_attention(q[None], kr[None], vr[None], attn_mask=mask)[0]
    torch.testing.assert_close(got, lib, rtol=1e-5, atol=1e-5)
    # plain attention without mask; one head; one key returns its value
    torch.testing.assert_close(plain.gqa_attention(q[:1], k[:1], v[:1], None),
                               F.scaled_dot_product_attention(q[None, :1], k[None, :1], v[None, :1])[0],
                               rtol=1e-5, atol=1e-5)
    one = plain.gqa_attention(q[:, :1], k[:, :1], v[:, :1], None)
    torch.testing.assert_close(one, repeat_kv(v[:, :1], nh // nkv))


def test_a_row_ignores_keys_after_its_position():
    nh, nkv, seq, start, d = 4, 2, 6, 2, 8
    q, k, v = torch.randn(nh, seq, d), torch.randn(nkv, start + seq, d), torch.randn(nkv, start + seq, d)
    mask = plain.causal_mask(seq, start)
    a = plain.gqa_attention(q, k, v, mask)
    k2, v2 = k.clone(), v.clone()
    k2[:, start + 3:], v2[:, start + 3:] = 9.0, -7.0      # perturb the keys rows 0..2 cannot see
    b = plain.gqa_attention(q, k2, v2, mask)
    assert torch.equal(a[:, :3], b[:, :3]) and not torch.equal(a[:, 3:], b[:, 3:])


def _model(cfg, seed=0):
    from rust_llm_inference_server_amd.registry import architecture_of
    from rust_llm_inference_server_amd.weights import random_weights
    arch = architecture_of(cfg)
    spec = arch.build_spec(arch.parse_config(cfg))
    w = random_weights(spec.tensor_specs(), seed, torch.float32)
    c = dict(cfg)
    c.setdefault("head_dim", cfg["hidden_size"] // cfg["num_attention_heads"])
    return w, c


def test_whole_model_prefix_property_and_position_shift():
    """Logits at position t depend on tokens 0..t only; and shifting all positions of the
    attention layer by a constant changes nothing, since only distances count."""
    w, c = _model(TINY_B)
    ids = torch.randint(0, c["vocab_size"], (20,)).tolist()
    full = plain.forward(w, c, ids)
    torch.testing.assert_close(plain.forward(w, c, ids[:11]), full[:11], rtol=1e-5, atol=1e-5)
    x = torch.randn(9, c["hidden_size"])
    inv = plain.inv_freqs(c["head_dim"], c["rope_theta"], c["rope_scaling"])
    a = plain.attention_layer(x, w, "model.layers.0.self_attn", c, inv, start_pos=0)
    b = plain.attention_layer(x, w, "model.layers.0.self_attn", c, inv, start_pos=13)
    torch.testing.assert_close(a, b, rtol=1e-4, atol=1e-5)


def test_tied_and_untied_heads():
    w, c = _model(TINY_A)                                  # tied: logits = h E^T
    ids = [3, 1, 4, 1, 5]
    logits = plain.forward(w, c, ids)
    assert logits.shape == (5, 256) and "lm_head.weight" not in w
    w2 = dict(w)
    w2["lm_head.weight"] = torch.zeros(256, 64)
    c2 = dict(c, tie_word_embeddings=False)
    assert plain.forward(w2, c2, ids).abs().max().item() == 0.0


def test_sampling_reference_vectors():
    assert plain.argmax(torch.tensor([0.1, 3.0, -1.0, 3.0])) == 1      # sampling.rs:184-199
    assert plain.argmax(torch.tensor([5.0, 1.0, 5.0, 0.0])) == 0
    assert plain.sample_row(torch.tensor([float("-inf"), -5.0]), 0, 0.0) == 1
    # repetition penalty [2, -2, 1], seen {0, 1}, p = 2 -> [1, -4, 1]  (sampler.rs:401-406)
    assert plain.apply_repetition_penalty([2.0, -2.0, 1.0], [0, 1, 1], 2.0) == [1.0, -4.0, 1.0]
    from rust_llm_inference_server_amd.sampling import lowbias32, row_key
    for x in (0, 1, 12345, 0xFFFFFFFF, 0x9E3779B9):
        assert plain.lowbias32(x) == lowbias32(x)
    assert plain.row_key((7 << 32) | 5, 11) == row_key((7 << 32) | 5, 11)
    assert plain.row_key(42, 1) != plain.row_key(42, 2)
    # the uniform is strictly inside (0, 1) at both ends of the hash range (sampling.rs:58-63)
    assert 0.0 < plain.uniform(0) < plain.uniform(0xFFFFFFFF) < 1.0


def test_gumbel_max_frequencies_follow_softmax():
    """sampling.rs:216-241: l = [0, 1, 2, -1], T = 0.7, keys row_key(42, i): frequencies equal
    softmax(l / T) within 0.015 (4,000 keys here, within 0.03)."""
    l = torch.tensor([0.0, 1.0, 2.0, -1.0])
    n = 4000
    counts = torch.zeros(4)
    for i in range(n):
        counts[plain.sample_row(l, plain.row_key(42, i), 1 / 0.7)] += 1
    assert (counts / n - torch.softmax(l / 0.7, 0)).abs().max().item() < 0.03


def test_perplexity_of_uniform_logits_is_the_vocabulary_size():
    """With an output head of zeros every logit is 0, every token costs ln(V): the perplexity
    is V and its standard error 0, whatever the tokens; and the count of scored tokens is
    windows * (ctx - 1 - ctx // 2)  (crates/engine/src/perplexity.rs:44-59)."""
    cfg = dict(TINY_B)
    g = torch.Generator().manual_seed(0)
    w = {}
    from rust_llm_inference_server_amd.registry import architecture_of
    arch = architecture_of(cfg)
    for spec in arch.build_spec(arch.parse_config(cfg)).tensor_specs():
        w[spec.name] = torch.randn(spec.shape, generator=g) * 0.05
    w["lm_head.weight"].zero_()
    c = dict(cfg)
    tokens = torch.randint(0, cfg["vocab_size"], (70,), generator=g).tolist()
    out = plain.perplexity(w, c, tokens, bos=1, ctx=16)
    assert out["windows"] == 4 and out["tokens_scored"] == 4 * 7
    assert abs(out["ppl"] - cfg["vocab_size"]) < 1e-6 * cfg["vocab_size"]
    assert out["ppl_stderr"] < 1e-4
    assert plain.perplexity(w, c, tokens, bos=1, ctx=16, max_windows=2)["windows"] == 2


def test_perplexity_replaces_each_windows_first_token_and_scores_its_second_half(tiny_folders):
    """crates/engine/src/perplexity.rs:44-59 written out by hand on a model whose logits depend on
    the tokens: windows of ctx tokens, the first token of each replaced by BOS, rows ctx/2 ..
    ctx-2 scored against the tokens that follow them.  What pins it: the value does not change
    with the token that BOS replaces, it does change with BOS (the later rows see it through
    attention), and it is neither the all-rows nor the unreplaced value."""
    w, c = plain.read_weights(tiny_folders["a"]), plain.read_config(tiny_folders["a"])
    g = torch.Generator().manual_seed(11)
    tokens = torch.randint(0, c["vocab_size"], (47,), generator=g).tolist()
    ctx, bos = 10, 7

    def by_hand(toks, first_row, replace):
        nll = []
        for wi in range(len(toks) // ctx):
            chunk = list(toks[wi * ctx:(wi + 1) * ctx])
            if replace:
                chunk[0] = bos
            logits = plain.forward(w, c, chunk).double()
            for row in range(first_row, ctx - 1):
                nll.append(float(torch.logsumexp(logits[row], 0) - logits[row][chunk[row + 1]]))
        return nll

    nll = by_hand(tokens, ctx // 2, True)
    assert len(nll) == 4 * 4                       # 4 windows (7 tokens left over), rows 5..8
    mean = sum(nll) / len(nll)
    out = plain.perplexity(w, c, tokens, bos=bos, ctx=ctx)
    assert out["windows"] == 4 and out["tokens_scored"] == 16
    assert abs(out["mean_nll"] - mean) < 1e-12 and abs(out["ppl"] - math.exp(mean)) < 1e-9
    var = sum(x * x for x in nll) / len(nll) - mean * mean
    assert abs(out["ppl_stderr"] - math.exp(mean) * math.sqrt(var / len(nll))) < 1e-9
    # the replaced tokens do not matter, BOS does
    other = list(tokens)
    for wi in range(4):
        other[wi * ctx] = (other[wi * ctx] + 1) % c["vocab_size"]
    assert plain.perplexity(w, c, other, bos=bos, ctx=ctx)["mean_nll"] == out["mean_nll"]
    assert abs(plain.perplexity(w, c, tokens, bos=bos + 1, ctx=ctx)["mean_nll"] - mean) > 1e-6
    # plausible mistakes give other numbers
    for wrong in (by_hand(tokens, ctx // 2, False), by_hand(tokens, 0, True),
                  by_hand(tokens, ctx // 2 + 1, True)):
        assert abs(sum(wrong) / len(wrong) - mean) > 1e-6
    # odd window length: rows 6 .. 11 of 13
    odd = plain.perplexity(w, c, tokens, bos=bos, ctx=13, max_windows=2)
    assert odd["windows"] == 2 and odd["tokens_scored"] == 2 * (13 - 1 - 13 // 2)


@pytest.mark.parametrize("name", ["a", "b", "c", "d"])
def test_the_two_plain_implementations_agree(tiny_folders, name):
    """The torch twin and the scalar-loop host implementation (plain_llama_host.cpp) were written
    apart from the same formulas: whole sequences through both, every logit within 1e-4 (the
    reference's own gate for its tiny model, crates/model/src/llama.rs:355).  A reading mistake
    would have to be made twice, the same way, to pass."""
    import plain_host
    if not plain_host.available():
        pytest.skip("g++ is not on the PATH")
    folder = tiny_folders[name]
    w, c = plain.read_weights(folder), plain.read_config(folder)
    g = torch.Generator().manual_seed(21)
    for n in (1, 2, 37):
        ids = torch.randint(0, c["vocab_size"], (n,), generator=g).tolist()
        a, b = plain.forward(w, c, ids), plain_host.forward(w, c, ids)
        assert a.shape == b.shape == (n, c["vocab_size"])
        assert (a - b).abs().max().item() < 1e-4
    # the llama3 bands of the two agree too (tiny b and d scale their frequencies)
    assert abs(b).max().item() > 0.05


# ------------------------------------------------- the whole model from library routines
def library_forward(w, c, ids, mistake=None):
    """The decoder of crates/model/src/llama.rs:264-286 put together from torch's own routines
    and nothing of plain_llama's but the inverse frequencies (pinned above by the reference's
    vector): ``F.embedding``, ``F.rms_norm``, ``F.linear``, ``F.silu``, the rotation as a
    multiplication of complex numbers (dims j and j + d/2 are the real and imaginary part,
    rope.rs:5-8) and ``F.scaled_dot_product_attention`` with its own causal mask and its own
    grouping of query heads (``enable_gqa``: query head h reads KV head h // group,
    attention.rs:240-245).  ``mistake`` builds a plausible misreading instead."""
    H, eps = c["hidden_size"], c["rms_norm_eps"]
    nh, nkv, d = c["num_attention_heads"], c["num_key_value_heads"], c["head_dim"]
    n = len(ids)
    angles = torch.outer(torch.arange(n, dtype=torch.float32),
                         plain.inv_freqs(d, c["rope_theta"], c.get("rope_scaling")))
    turn = torch.polar(torch.ones_like(angles), angles)[:, None, :]           # e^(i p f_j)

    def rotate(t):                                                             # (n, heads, d)
        z = torch.complex(t[..., :d // 2].contiguous(), t[..., d // 2:].contiguous()) * turn
        return torch.cat([z.real, z.imag], dim=-1)

    def norm(x, name):
        return F.rms_norm(x, (H,), w[name], eps)

    x = F.embedding(torch.tensor(ids), w["model.embed_tokens.weight"])
    for layer in range(c["num_hidden_layers"]):
        p = f"model.layers.{layer}"

        def mixer(h):
            q = rotate(F.linear(h, w[f"{p}.self_attn.q_proj.weight"]).view(n, nh, d))
            k = rotate(F.linear(h, w[f"{p}.self_attn.k_proj.weight"]).view(n, nkv, d))
            v = F.linear(h, w[f"{p}.self_attn.v_proj.weight"]).view(n, nkv, d)
            a = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None],
                                               v.transpose(0, 1)[None], is_causal=True,
                                               enable_gqa=True)[0]
            return F.linear(a.transpose(0, 1).reshape(n, nh * d), w[f"{p}.self_attn.o_proj.weight"])

        def feed_forward(h):
            return F.linear(F.silu(F.linear(h, w[f"{p}.mlp.gate_proj.weight"]))
                            * F.linear(h, w[f"{p}.mlp.up_proj.weight"]), w[f"{p}.mlp.down_proj.weight"])

        first, second = f"{p}.input_layernorm.weight", f"{p}.post_attention_layernorm.weight"
        if mistake == "post-norm":                      # norm after the residual add
            x = norm(x + mixer(x), first)
            x = norm(x + feed_forward(x), second)
        elif mistake == "parallel":                     # both parts read the same stream
            x = x + mixer(norm(x, first)) + feed_forward(norm(x, second))
        elif mistake == "one residual":                 # the feed-forward's input is not added back
            x = x + mixer(norm(x, first))
            x = feed_forward(norm(x, second))
        elif mistake == "norms swapped":
            x = x + mixer(norm(x, second))
            x = x + feed_forward(norm(x, first))
        else:                                           # llama.rs:264-279
            x = x + mixer(norm(x, first))
            x = x + feed_forward(norm(x, second))
    if mistake != "no final norm":
        x = norm(x, "model.norm.weight")                # llama.rs:280-283
    head = "model.embed_tokens.weight" if c.get("tie_word_embeddings") else "lm_head.weight"
    return F.linear(x, w[head])


@pytest.mark.parametrize("name", ["a", "b", "c", "d"])
def test_the_whole_model_reduces_to_library_routines(tiny_folders, name):
    """Block order, the two residual adds, the final norm in front of the head, the rotation's
    pairing and sign, the grouping of heads and the causal mask, all at once, against a model
    assembled from the library's routines (each of which is documented on its own): every logit
    of a 40-token sequence within 1e-5 for the four tiny configurations (tied and untied heads,
    scaled and unscaled frequencies, head_dim * heads != hidden, one KV head for several
    queries).  The norm weights are 1 + N(0, 0.02) and are spread further here, so that a norm
    in the wrong place or a missing one shows; each plausible misreading moves the logits by
    more than a hundred times the gate.  (The reference holds its model against the
    ``transformers`` package, scripts/parity/dump_reference.py:99-154; that package's model
    code is not imported here, so the pin is to the library routines the formulas reduce to.)"""
    w, c = plain.read_weights(tiny_folders[name]), plain.read_config(tiny_folders[name])
    g = torch.Generator().manual_seed(5)
    w = dict(w)
    for k in w:
        if k.endswith("norm.weight"):
            w[k] = w[k] + 0.5 * torch.rand(w[k].shape, generator=g)
    ids = torch.randint(0, c["vocab_size"], (40,), generator=g).tolist()
    mine, want = plain.forward(w, c, ids), library_forward(w, c, ids)
    assert mine.shape == want.shape == (40, c["vocab_size"])
    assert (mine - want).abs().max().item() < 1e-5
    assert want.abs().max().item() > 0.05
    for mistake in ("post-norm", "parallel", "one residual", "norms swapped", "no final norm"):
        wrong = library_forward(w, c, ids, mistake)
        assert (mine - wrong).abs().max().item() > 1e-3, mistake
    # one token at position 0 sees itself only: the attention returns its value, rotation or not
    one = plain.forward(w, c, ids[:1])
    assert (one - want[:1]).abs().max().item() < 1e-5
