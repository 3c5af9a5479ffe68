"""The parts alone, and models put together from them in ways the Llama decoder does not use:
a layer with a window beside layers without, a layer named twice in the run order, a layer
that reads another layer's cache, and a toy mixer with state of its own that the test defines
and registers without touching the package.  Everything runs on the GPU against plain code."""
import math

import pytest
import torch

import plain_llama as plain
import traces
from conftest import TINY_B

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def ctx_for(weights, dtype=torch.float32, max_positions=256):
    from rust_llm_inference_server_amd.parts import BuildContext
    return BuildContext(device=DEV, act_dtype=dtype, max_positions=max_positions,
                        weights={k: v.to(DEV) for k, v in weights.items()})


# --------------------------------------------------------------- each part alone
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part(dtype):
    from rust_llm_inference_server_amd.parts import PartSpec, ResidualStream, create
    w = {"n.weight": 1 + 0.1 * torch.randn(100)}
    norm = create("norm", PartSpec("rmsnorm", {"size": 100, "eps": 1e-6}), "n", ctx_for(w, dtype))
    x, d = torch.randn(6, 100), torch.randn(6, 100).to(dtype)
    stream = ResidualStream(x.to(DEV).clone())
    stream.add(d.to(DEV))
    y = norm.forward(stream)
    assert stream.pending is None and y.dtype == dtype
    want_x = x + d.float()
    torch.testing.assert_close(stream.x.cpu(), want_x, atol=1e-6, rtol=1e-6)   # 32-bit residual
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    torch.testing.assert_close(y.float().cpu(), plain.rms_norm(want_x, w["n.weight"], 1e-6),
                               atol=tol, rtol=tol)
    rows = torch.tensor([4, 1], dtype=torch.int32, device=DEV)
    stream.add(d.to(DEV))
    y2 = norm.forward_rows(stream, rows)
    want2 = plain.rms_norm((want_x + d.float())[[4, 1]], w["n.weight"], 1e-6)
    torch.testing.assert_close(y2.float().cpu(), want2, atol=tol, rtol=tol)


def test_position_part_tables():
    from rust_llm_inference_server_amd.parts import PartSpec, create
    sc = TINY_B["rope_scaling"]
    rope = create("position", PartSpec("rope", {"rot_dim": 32, "theta": 500000.0, "scaling": sc}),
                  "", ctx_for({}, max_positions=200))
    cos, sin = plain.rope_tables(plain.inv_freqs(32, 500000.0, sc), range(200))
    assert rope.cos.dtype == torch.float32 and rope.cos.shape == (200, 16)
    torch.testing.assert_close(rope.cos.cpu(), cos, atol=1e-6, rtol=0)
    torch.testing.assert_close(rope.sin.cpu(), sin, atol=1e-6, rtol=0)
    with pytest.raises(ValueError, match="unknown scaling"):
        create("position", PartSpec("rope", {"rot_dim": 32, "theta": 1e4,
                                             "scaling": {"rope_type": "yarn"}}), "", ctx_for({}))


def test_a_pending_projection_meets_the_norm_behind_it():
    """A mixer's or feed-forward's last projection may reach the residual stream not yet run
    (``ops.pending_linear``).  A norm whose consumer takes the norm into its own kernel then
    runs the projection with the residual add inside and hands rows and sums of squares to the
    consumer's product; any other taker (a plain norm, a norm over selected rows, a flush) gets
    the tensor.  Every way ends with the same residual and, within the bfloat16 tolerance, the
    same normalised product."""
    from rust_llm_inference_server_amd import ops
    from rust_llm_inference_server_amd.parts import PartSpec, ResidualStream, create
    from rust_llm_inference_server_amd.parts.base import NormedInput, as_tensor
    dtype = torch.bfloat16
    H, K, N, T = 192, 320, 400, 9
    w = {"n.weight": 1 + 0.1 * torch.randn(H)}
    norm = create("norm", PartSpec("rmsnorm", {"size": H, "eps": 1e-6}), "n", ctx_for(w, dtype))
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(T, K, generator=g) * 0.5).to(dtype).to(DEV)
    w1 = (torch.randn(H, K, generator=g) * 0.05).to(dtype).to(DEV)
    w2 = (torch.randn(N, H, generator=g) * 0.05).to(dtype).to(DEV)
    resid = torch.randn(T, H, generator=g).to(DEV)
    delta = (x.float() @ w1.float().t()).to(dtype).float()
    want_resid = resid + delta
    want = plain.rms_norm(want_resid.cpu(), w["n.weight"], 1e-6) @ w2.float().cpu().t()

    def stream_with_pending():
        stream = ResidualStream(resid.clone(), dtype)
        pending = ops.pending_linear(x, w1, dtype)
        assert isinstance(pending, ops.PendingProduct)
        stream.add(pending)
        return stream

    calls = []
    real = ops.linear_join_norm
    ops.linear_join_norm = lambda *a: calls.append(1) or real(*a)
    try:
        stream = stream_with_pending()
        joined = NormedInput(norm, stream).linear(w2, dtype)
    finally:
        ops.linear_join_norm = real
    assert calls and stream.pending is None
    torch.testing.assert_close(stream.x, want_resid, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(joined.float().cpu(), want, atol=3e-2, rtol=3e-2)
    stream = stream_with_pending()
    plainly = ops.linear(norm.forward(stream), w2, dtype)           # a norm that stands alone
    torch.testing.assert_close(stream.x, want_resid, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(plainly.float(), joined.float(), atol=3e-2, rtol=3e-2)
    stream = stream_with_pending()
    rows = torch.tensor([4, 1], dtype=torch.int32, device=DEV)
    some = norm.forward_rows(stream, rows)                          # leaves the residual alone
    assert isinstance(stream.pending, torch.Tensor)
    torch.testing.assert_close(ops.linear(some, w2, dtype).float(), joined.float()[[4, 1]], atol=3e-2, rtol=3e-2)
    torch.testing.assert_close(stream.flush(), want_resid, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(as_tensor(ops.pending_linear(x, w1, dtype)).float(), delta, atol=0, rtol=0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forward_embedding_and_head_parts(dtype):
    from rust_llm_inference_server_amd.parts import PartSpec, create
    H, I, V = 72, 200, 131
    w = {"m.gate_proj.weight": torch.randn(I, H) * 0.1, "m.up_proj.weight": torch.randn(I, H) * 0.1,
         "m.down_proj.weight": torch.randn(H, I) * 0.1, "e.weight": torch.randn(V, H),
         "h.weight": torch.randn(V, H) * 0.1}
    w = {k: v.to(dtype) for k, v in w.items()}
    ctx = ctx_for(w, dtype)
    mlp = create("feed_forward", PartSpec("swiglu", {"hidden_size": H, "intermediate_size": I}), "m", ctx)
    x = torch.randn(9, H).to(dtype)
    wf = {k: v.float() for k, v in w.items()}
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    from rust_llm_inference_server_amd.parts.base import as_tensor
    torch.testing.assert_close(as_tensor(mlp.forward(x.to(DEV), None)).float().cpu(),
                               plain.swiglu_mlp(x.float(), wf, "m"), atol=tol, rtol=tol)
    emb = create("embedding", PartSpec("token", {"vocab_size": V, "hidden_size": H}), "e", ctx)
    ids = [5, 130, 0, 5]
    out = emb.forward(torch.tensor(ids, dtype=torch.int32, device=DEV))
    assert out.dtype == torch.float32
    torch.testing.assert_close(out.cpu(), plain.embedding(wf["e.weight"], ids), atol=0, rtol=0)
    for tied in (None, "e.weight"):
        head = create("head", PartSpec("linear", {"vocab_size": V, "hidden_size": H, "tied_to": tied}),
                      "h", ctx)
        logits = head.forward(x.to(DEV))
        assert logits.dtype == torch.float32
        torch.testing.assert_close(logits.cpu(), plain.linear(x.float(), wf[tied or "h.weight"]),
                                   atol=tol * 10, rtol=tol)


# --------------------------------------------------- models built from a ModelSpec
def layer_spec(H, nh, nkv, d, I, eps, theta, window, mixer="attention", extra=None):
    from rust_llm_inference_server_amd.parts import PartSpec
    norm = PartSpec("rmsnorm", {"size": H, "eps": eps})
    mixer_params = {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d,
                    "scale": 1 / math.sqrt(d), "window": window,
                    "position": PartSpec("rope", {"rot_dim": d, "theta": theta, "scaling": None})}
    if extra:
        mixer_params = extra
    return PartSpec("prenorm", {
        "mixer": PartSpec(mixer, mixer_params),
        "feed_forward": PartSpec("swiglu", {"hidden_size": H, "intermediate_size": I}),
        "mixer_norm": norm, "ffn_norm": norm,
        "names": {"mixer_norm": "input_layernorm", "mixer": "self_attn",
                  "ffn_norm": "post_attention_layernorm", "feed_forward": "mlp"}})


def toy_spec(blocks, run_order=None, H=64, V=97):
    from rust_llm_inference_server_amd.models import LayerSpec, ModelSpec
    from rust_llm_inference_server_amd.parts import PartSpec
    return ModelSpec(
        hidden_size=H, vocab_size=V,
        embedding=PartSpec("token", {"vocab_size": V, "hidden_size": H}),
        embedding_prefix="model.embed_tokens",
        layers=[LayerSpec(b, f"model.layers.{i}") for i, b in enumerate(blocks)],
        final_norm=PartSpec("rmsnorm", {"size": H, "eps": 1e-5}), final_norm_prefix="model.norm",
        head=PartSpec("linear", {"vocab_size": V, "hidden_size": H, "tied_to": None}),
        head_prefix="lm_head", run_order=run_order)


def plain_toy_forward(w, ids, layers, runs, H=64, eps=1e-5, theta=1e4):
    """Whole-sequence forward of the toy models: ``layers`` is a list of dicts
    (nh, nkv, d, window), ``runs`` a list of (layer, cache_of) like the run order."""
    x = plain.embedding(w["model.embed_tokens.weight"], ids)
    T = len(ids)
    kv_of_run = {}
    for r, (li, cache_of) in enumerate(runs):
        L, p = layers[li], f"model.layers.{li}"
        h = plain.rms_norm(x, w[f"{p}.input_layernorm.weight"], eps)
        nh, nkv, d = L["nh"], L["nkv"], L["d"]
        inv = plain.inv_freqs(d, theta, None)
        cos, sin = plain.rope_tables(inv, range(T))
        q = plain.linear(h, w[f"{p}.self_attn.q_proj.weight"]).reshape(T, nh, d).transpose(0, 1)
        q = plain.rope_apply(q, cos, sin)
        if cache_of is None:
            k = plain.linear(h, w[f"{p}.self_attn.k_proj.weight"]).reshape(T, nkv, d).transpose(0, 1)
            v = plain.linear(h, w[f"{p}.self_attn.v_proj.weight"]).reshape(T, nkv, d).transpose(0, 1)
            kv_of_run[r] = (plain.rope_apply(k, cos, sin), v)
        k, v = kv_of_run[r if cache_of is None else cache_of]
        o = plain.gqa_attention(q, k, v, plain.causal_mask(T, 0, L["window"]))
        x = x + plain.linear(o.transpose(0, 1).reshape(T, nh * d), w[f"{p}.self_attn.o_proj.weight"])
        h = plain.rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], eps)
        x = x + plain.swiglu_mlp(h, w, f"{p}.mlp")
    return plain.linear(plain.rms_norm(x, w["model.norm.weight"], eps), w["lm_head.weight"])


def run_families(spec, weights, dtype, reqs, ref, tol, page_size=8, check_window_pages=False):
    from rust_llm_inference_server_amd.engine import ModelRunner
    from rust_llm_inference_server_amd.models import Model
    tdt = torch.float32 if dtype == "float32" else torch.bfloat16
    for build in (traces.trace_whole, traces.trace_tail, traces.trace_portions, traces.trace_mixed):
        steps, max_tokens = build(reqs)
        model = Model(spec, {k: v.to(tdt).to(DEV) for k, v in weights.items()}, tdt, DEV, 256)
        runner = ModelRunner(model, num_pages=max_tokens // page_size, page_size=page_size,
                             max_num_seqs=8)
        outputs = traces.replay_in_process(runner, steps)
        got = traces.collect(steps, outputs, spec.vocab_size)
        for k, tokens in reqs.items():
            mine = torch.stack([got[k][p] for p in range(len(tokens))])
            diff = (mine - ref[k]).abs().max(dim=-1).values
            bad = (diff > tol).nonzero()
            assert bad.numel() == 0, (f"{build.__name__} request {k}: first wrong position "
                                      f"{int(bad[0])} (|diff| {diff[bad[0]].item():.3e})")
        for g in range(runner.cache.num_groups):
            assert runner.cache.num_free_pages(g) == runner.cache.num_pages(g)
    return runner


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-4), ("bfloat16", 3e-2)])
def test_window_layers_beside_full_layers(dtype, tol):
    """Layer 0 sees every earlier position, layer 1 only the last 24, layer 2 the last 5 (less
    than a page): three page groups; windowed groups give pages back while a request runs."""
    from rust_llm_inference_server_amd.weights import random_weights
    layers = [dict(nh=4, nkv=2, d=16, window=None), dict(nh=4, nkv=2, d=16, window=24),
              dict(nh=2, nkv=1, d=32, window=5)]
    spec = toy_spec([layer_spec(64, L["nh"], L["nkv"], L["d"], 96, 1e-5, 1e4, L["window"]) for L in layers])
    tdt = torch.float32 if dtype == "float32" else torch.bfloat16
    w = {k: v.to(tdt).float() for k, v in random_weights(spec.tensor_specs(), 3, torch.float32).items()}
    # sharpen attention so that a key just outside a window would be seen if it leaked in
    for i in range(3):
        w[f"model.layers.{i}.self_attn.q_proj.weight"] *= 8
        w[f"model.layers.{i}.self_attn.k_proj.weight"] *= 8
    w = {k: v.to(tdt).float() for k, v in w.items()}
    reqs = traces.random_requests(97, [70, 9, 130, 33, 2, 64], seed=5)
    runs = [(0, None), (1, None), (2, None)]
    ref = {k: plain_toy_forward(w, t, layers, runs) for k, t in reqs.items()}
    runner = run_families(spec, w, dtype, reqs, ref, tol)
    assert [g.window for g in runner.cache.groups] == [None, 24, 5]
    # pages of the windowed groups return while the request is alive
    runner.reserve(0, 100)
    from rust_llm_inference_server_amd.engine import StepEntry
    runner.step([StepEntry(0, reqs["r2"][:100], [])])
    free = [runner.cache.num_free_pages(g) for g in range(3)]
    assert free[0] < free[1] < free[2]
    runner.cache.check_invariants()


def test_engine_sizes_the_pools_of_windowed_layers_by_their_windows():
    """An engine over full and windowed layers, its pools cut from one budget of bytes: the
    windowed groups get what ``max_num_seqs`` requests can hold of them (but room for one
    request of the longest length, which admission reserves whole), the group that keeps
    everything gets the rest.  Requests longer than the windows, prompts in portions, more
    requests than seats: every greedy token is the plain implementation's, the windowed pools
    never run dry, and every page comes back."""
    from rust_llm_inference_server_amd.config import EngineConfig
    from rust_llm_inference_server_amd.engine import Engine
    from rust_llm_inference_server_amd.models import Model
    from rust_llm_inference_server_amd.sampling import SamplingParams
    from rust_llm_inference_server_amd.weights import random_weights
    layers = [dict(nh=4, nkv=2, d=16, window=None), dict(nh=4, nkv=2, d=16, window=24),
              dict(nh=2, nkv=1, d=32, window=5)]
    spec = toy_spec([layer_spec(64, L["nh"], L["nkv"], L["d"], 96, 1e-5, 1e4, L["window"]) for L in layers])
    w = random_weights(spec.tensor_specs(), 3, torch.float32)
    model = Model(spec, {k: v.to(DEV) for k, v in w.items()}, torch.float32, DEV, 256)
    per_page = 64 * 4 * 8                                  # K and V of one layer, a page of 8
    engine = Engine(model, EngineConfig(kv_cache_gb=100 * 3 * per_page / (1 << 30), block_size=8,
                                        max_num_seqs=4, max_batched_tokens=32, max_seq_len=256))
    cache = engine.runner.cache
    pools = [cache.num_pages(g) for g in range(3)]
    # window 24: 4 x (ceil((24 + 32) / 8) + 1) = 32 pages, window 5: 4 x 6 = 24; one request of
    # 256 positions needs 33 either way; the rest of 300 pages' worth of bytes goes to group 0
    assert pools == [300 - 2 * 33, 33, 33]
    assert [t.shape[1] for g in engine.runner.pools.arrays for t in g.values()] == \
        [pools[0] + 1] * 2 + [34] * 4
    assert engine.max_seq_len == (33 - 1) * 8
    g = torch.Generator().manual_seed(9)
    lengths, new = [70, 9, 130, 33, 200, 2, 51], 14
    prompts = [torch.randint(0, 97, (n,), generator=g).tolist() for n in lengths]
    low = [cache.num_pages(i) for i in range(3)]
    ids = [engine.add_request(p, SamplingParams.greedy(new)) for p in prompts]
    while engine.has_work():
        engine.step()
        low = [min(a, cache.num_free_pages(i)) for i, a in enumerate(low)]
        cache.check_invariants()
    runs = [(0, None), (1, None), (2, None)]
    for p, i in zip(prompts, ids):
        got = engine.pop_finished(i)
        assert got.finish_reason == "length"
        tokens = list(p)
        for t in got.token_ids:
            logits = plain_toy_forward(w, tokens, layers, runs)[-1]
            assert int(torch.argmax(logits)) == t, (len(p), len(tokens))
            tokens.append(t)
    assert [cache.num_free_pages(i) for i in range(3)] == pools
    # the windowed pools were used hard (admission reserves whole prompts there) but held
    assert low[1] < 16 and low[2] < 16 and low[0] > 100, low
    assert engine.stats().preemptions == 0


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-4), ("bfloat16", 3e-2)])
def test_run_order_names_a_layer_twice_and_shares_a_cache(dtype, tol):
    """Run order: layer 0, layer 1, layer 0 again (a second cache of its own), then layer 1
    reading the cache its first run wrote (it writes nothing)."""
    from rust_llm_inference_server_amd.models import RunEntry
    from rust_llm_inference_server_amd.weights import random_weights
    layers = [dict(nh=4, nkv=1, d=16, window=None), dict(nh=3, nkv=3, d=16, window=None)]
    order = [RunEntry(0), RunEntry(1), RunEntry(0), RunEntry(1, cache_of=1)]
    spec = toy_spec([layer_spec(64, L["nh"], L["nkv"], L["d"], 80, 1e-5, 1e4, None) for L in layers],
                    run_order=order)
    tdt = torch.float32 if dtype == "float32" else torch.bfloat16
    w = {k: v.to(tdt).float() for k, v in random_weights(spec.tensor_specs(), 4, torch.float32).items()}
    reqs = traces.random_requests(97, [40, 5, 90, 17], seed=6)
    runs = [(0, None), (1, None), (0, None), (1, 1)]
    ref = {k: plain_toy_forward(w, t, layers, runs) for k, t in reqs.items()}
    from rust_llm_inference_server_amd.models import Model
    model = Model(spec, {k: v.to(DEV) for k, v in w.items()}, torch.float32, DEV, 256)
    assert [len(g.writer_runs) for g in model.cache_groups] == [2, 1]
    assert [(b.group, b.slot, b.writes) for b in model.bindings] == \
        [(0, 0, True), (1, 0, True), (0, 1, True), (1, 0, False)]
    run_families(spec, w, dtype, reqs, ref, tol)
    from rust_llm_inference_server_amd.models import ModelSpec
    bad = toy_spec([layer_spec(64, 4, 1, 16, 80, 1e-5, 1e4, None)] * 2,
                   run_order=[RunEntry(0, cache_of=1), RunEntry(1)])
    with pytest.raises(ValueError, match="does not run before"):
        bad.validate()


# ------------------------------------------------ a toy mixer with state of its own
def register_toy():
    """Defined and registered here, in the test: a mixer whose memory of the past is one
    vector per request, the running sum of its inputs (kept in the request's state slot)."""
    from rust_llm_inference_server_amd.parts import Mixer, TensorSpec, register
    from rust_llm_inference_server_amd.parts.base import join

    @register("mixer", "toy_running_sum")
    class RunningSum(Mixer):
        @classmethod
        def tensor_specs(cls, params, prefix):
            return [TensorSpec(join(prefix, "mix.weight"), (params["hidden_size"],) * 2)]

        def __init__(self, params, prefix, ctx):
            super().__init__(params, prefix, ctx)
            self.size = params["hidden_size"]
            self.weight = ctx.take(join(prefix, "mix.weight")).float()
            self.decay = float(params["decay"])
            self.act_dtype = ctx.act_dtype
            # With "on_device" a step of one token per request is device work alone (the
            # state rows are gathered and scattered by the step's slot ids), so that such steps
            # may be captured into a graph.
            self.graph_safe = bool(params.get("on_device", False))

        def state_bytes(self):
            return 4 * self.size

        def forward(self, x, step, binding):
            if self.graph_safe and step.all_decode:
                states = binding.state.view(torch.float32)          # (slots, size)
                slots = step.state_slots[:x.shape[0]].long()
                new = states.index_select(0, slots) * self.decay + x.float()
                states.index_copy_(0, slots, new)
                return (new @ self.weight.t()).to(self.act_dtype)
            out = torch.empty_like(x, dtype=torch.float32)
            begin = 0
            for n, slot in zip(step.host_new, step.host_state_slots):
                state = binding.state[slot].view(torch.float32)
                for t in range(begin, begin + n):            # in order, token by token
                    state.mul_(self.decay).add_(x[t].float())
                    out[t] = state
                begin += n
            return (out @ self.weight.t()).to(self.act_dtype)

    return RunningSum


def plain_running_sum_model(w, ids, layers, H=48, eps=1e-5, decay=0.9):
    x = plain.embedding(w["model.embed_tokens.weight"], ids)
    T = len(ids)
    for li, kind in enumerate(layers):
        p = f"model.layers.{li}"
        h = plain.rms_norm(x, w[f"{p}.input_layernorm.weight"], eps)
        if kind == "toy":
            s, rows = torch.zeros(H), []
            for t in range(T):
                s = s * decay + h[t]
                rows.append(s)
            x = x + torch.stack(rows) @ w[f"{p}.self_attn.mix.weight"].t()
        else:
            cfg = {"num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 16}
            x = x + plain.attention_layer(h, w, f"{p}.self_attn", cfg, plain.inv_freqs(16, 1e4, None))
        h = plain.rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], eps)
        x = x + plain.swiglu_mlp(h, w, f"{p}.mlp")
    return plain.linear(plain.rms_norm(x, w["model.norm.weight"], eps), w["lm_head.weight"])


def test_toy_mixer_with_state_registers_builds_and_steps(tmp_path):
    """A new mixer kind and a new architecture name, both registered from the test; the model
    folder is loaded through the ordinary loader and replayed in every way of cutting, with
    fewer state slots than requests so that slots (and their stale contents) are used again."""
    from rust_llm_inference_server_amd.engine import ModelRunner, load_model
    from rust_llm_inference_server_amd.registry import Architecture, register_architecture
    from rust_llm_inference_server_amd.weights import write_model_folder
    register_toy()
    H = 48
    kinds = ["toy", "attention", "toy"]

    def build_spec(cfg):
        blocks = []
        for kind in cfg["mixers"]:
            if kind == "toy":
                blocks.append(layer_spec(H, 1, 1, 16, 64, 1e-5, 1e4, None, mixer="toy_running_sum",
                                         extra={"hidden_size": H, "decay": 0.9}))
            else:
                blocks.append(layer_spec(H, 3, 1, 16, 64, 1e-5, 1e4, None))
        return toy_spec(blocks, H=H, V=cfg["vocab_size"])

    register_architecture(Architecture("ToyForCausalLM", parse_config=lambda d: d,
                                       build_spec=build_spec, config_to_dict=lambda c: c))
    config = {"architectures": ["ToyForCausalLM"], "vocab_size": 97, "mixers": kinds}
    spec = build_spec(config)
    folder = str(tmp_path / "toy")
    write_model_folder(folder, config, spec.tensor_specs(), seed=9)
    w = plain.read_weights(folder)
    reqs = traces.random_requests(97, [30, 4, 70, 11, 45, 2], seed=8)
    ref = {k: plain_running_sum_model(w, t, kinds) for k, t in reqs.items()}
    for build in (traces.trace_whole, traces.trace_tail, traces.trace_portions, traces.trace_mixed):
        steps, max_tokens = build(reqs)
        model = load_model(folder, "float32", max_positions=128)
        assert model.state_bytes == 2 * 4 * H and len(model.cache_groups) == 1
        runner = ModelRunner(model, num_pages=max_tokens // 16, page_size=16, max_num_seqs=4)
        assert runner.cache.num_state_slots == 4          # 6 requests share 4 slots over time
        got = traces.collect(steps, traces.replay_in_process(runner, steps), 97)
        for k, tokens in reqs.items():
            mine = torch.stack([got[k][p] for p in range(len(tokens))])
            assert (mine - ref[k]).abs().max().item() < 2e-4, f"{build.__name__} request {k}"
        assert runner.cache.num_free_slots() == 4


def test_toy_mixer_with_state_through_captured_decode_steps(tmp_path, monkeypatch):
    """The same toy mixer doing its single-token steps on the device alone, so that the model's
    decode steps are captured into HIP graphs: every way of cutting, then requests that start
    with single tokens on state slots that earlier requests left full.  The captured path must
    clear the slot of a request that starts, keep padding rows off the live slots, and not
    advance any state while it captures."""
    from rust_llm_inference_server_amd.engine import ModelRunner, StepEntry, load_model
    from rust_llm_inference_server_amd.registry import Architecture, register_architecture
    from rust_llm_inference_server_amd.weights import write_model_folder
    register_toy()
    H = 48
    kinds = ["toy", "attention", "toy"]

    def build_spec(cfg):
        blocks = []
        for kind in cfg["mixers"]:
            if kind == "toy":
                blocks.append(layer_spec(H, 1, 1, 16, 64, 1e-5, 1e4, None, mixer="toy_running_sum",
                                         extra={"hidden_size": H, "decay": 0.9, "on_device": True}))
            else:
                blocks.append(layer_spec(H, 3, 1, 16, 64, 1e-5, 1e4, None))
        return toy_spec(blocks, H=H, V=cfg["vocab_size"])

    register_architecture(Architecture("ToyOnDeviceForCausalLM", parse_config=lambda d: d,
                                       build_spec=build_spec, config_to_dict=lambda c: c))
    config = {"architectures": ["ToyOnDeviceForCausalLM"], "vocab_size": 97, "mixers": kinds}
    folder = str(tmp_path / "toy")
    write_model_folder(folder, config, build_spec(config).tensor_specs(), seed=9)
    w = plain.read_weights(folder)
    reqs = traces.random_requests(97, [30, 4, 70, 11, 45, 2], seed=8)
    ref = {k: plain_running_sum_model(w, t, kinds) for k, t in reqs.items()}
    for build in (traces.trace_whole, traces.trace_tail, traces.trace_portions, traces.trace_mixed):
        steps, max_tokens = build(reqs)
        model = load_model(folder, "float32", max_positions=128)
        assert model.graph_safe and model.state_bytes == 2 * 4 * H
        runner = ModelRunner(model, num_pages=max_tokens // 16, page_size=16, max_num_seqs=4)
        assert runner.use_graphs
        got = traces.collect(steps, traces.replay_in_process(runner, steps), 97)
        if build in (traces.trace_tail, traces.trace_mixed):
            assert runner._graphs, "no decode step took the graph path"
        for k, tokens in reqs.items():
            mine = torch.stack([got[k][p] for p in range(len(tokens))])
            assert (mine - ref[k]).abs().max().item() < 2e-4, f"{build.__name__} request {k}"
        assert runner.cache.num_free_slots() == 4
    # Requests fed one token at a time from position 0, three at once in a bucket of four (one
    # padding row), on slots that the requests above left full; a fourth joins later, when the
    # graph exists already.
    keys = ["r0", "r2", "r4", "r3"]
    for i, k in enumerate(keys[:3]):
        runner.reserve(100 + i, 12)
    runner.reserve(103, 8)
    for t in range(12):
        live = [0, 1, 2] + ([3] if t >= 4 else [])
        entries = [StepEntry(100 + i, [reqs[keys[i]][t - (4 if i == 3 else 0)]], [0]) for i in live]
        logits = runner.step(entries).float().cpu()
        for row, i in enumerate(live):
            pos = t - (4 if i == 3 else 0)
            assert (logits[row] - ref[keys[i]][pos]).abs().max().item() < 2e-4, (keys[i], pos)
    assert {1 << 2} <= set(runner._graphs)
    for i in range(4):
        runner.free(100 + i)
    # Prompt steps whose shape comes back are captured too.  Off the decode path this mixer
    # works through the state slots in a host loop, so a captured step holds its slot for
    # good: the slot is part of a step's shape, and a request on another slot (a bystander
    # holds the first one meanwhile) is another shape with a capture of its own.  The slot
    # of a request that starts is cleared outside the captured step.
    from rust_llm_inference_server_amd.engine.graph import RepeatedSteps
    monkeypatch.setattr(RepeatedSteps, "CAPTURE_AT", 2)
    for r in range(8):
        if r == 4:
            runner.reserve(300, 3)
            runner.step([StepEntry(300, reqs["r0"][:3], [])])
        k = ("r2", "r4")[r % 2]
        runner.reserve(200 + r, 20)
        first = runner.step([StepEntry(200 + r, reqs[k][:9], [8])]).float().cpu()
        second = runner.step([StepEntry(200 + r, reqs[k][9:20], [0, 10])]).float().cpu()
        runner.free(200 + r)
        for got_row, pos in ((first[0], 8), (second[0], 9), (second[1], 19)):
            assert (got_row - ref[k][pos]).abs().max().item() < 2e-4, (r, k, pos)
    assert len(runner._repeated.graphs) == 4 and runner._repeated.replays == 12


# ------------------------- a toy mixer that caches one vector per position
def register_latent_toy():
    """Defined and registered here, in the test: a mixer whose memory of the past grows with
    the length but is no pair of keys and values.  It keeps one latent vector of ``rank``
    numbers per position in pages of its own kind and gives every token the mean of the latents
    up to and including its own, projected back up.  The latents are cached in float32 whatever
    the model's activation dtype is: the page array names its own dtype."""
    from rust_llm_inference_server_amd.parts import Mixer, TensorSpec, register
    from rust_llm_inference_server_amd.parts.base import PAGE, CacheRequest, PageArray, join

    @register("mixer", "toy_latent_mean")
    class LatentMean(Mixer):
        @classmethod
        def tensor_specs(cls, params, prefix):
            H, r = params["hidden_size"], params["rank"]
            return [TensorSpec(join(prefix, "down.weight"), (r, H)),
                    TensorSpec(join(prefix, "up.weight"), (H, r))]

        def __init__(self, params, prefix, ctx):
            super().__init__(params, prefix, ctx)
            self.rank = params["rank"]
            self.down = ctx.take(join(prefix, "down.weight")).float()
            self.up = ctx.take(join(prefix, "up.weight")).float()
            self.act_dtype = ctx.act_dtype

        def cache_request(self):
            return CacheRequest((PageArray("latent", (PAGE, self.rank), dtype=torch.float32),))

        def forward(self, x, step, binding):
            group = step.groups[binding.group]
            pages = binding.pages["latent"]                       # (num pages, page, rank)
            ps = group.page_size
            flat = pages.view(-1, self.rank)
            latent = (x.float() @ self.down.t()).to(pages.dtype)
            if binding.writes:
                flat.index_copy_(0, group.slots.long(), latent)
            tables = group.block_tables.cpu()
            out = torch.empty((x.shape[0], self.rank), dtype=torch.float32, device=x.device)
            begin = 0
            for s, (start, n) in enumerate(zip(step.host_start_pos, step.host_new)):
                pos = torch.arange(start + n)
                rows = (tables[s, pos // ps].long() * ps + pos % ps).to(x.device)
                seen = flat.index_select(0, rows).float().cumsum(0)       # read back from the pages
                count = torch.arange(1, start + n + 1, device=x.device).unsqueeze(1)
                out[begin:begin + n] = (seen / count)[start:]
                begin += n
            return (out @ self.up.t()).to(self.act_dtype)

    return LatentMean


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-4), ("bfloat16", 3e-2)])
def test_toy_mixer_with_a_cache_kind_of_its_own(tmp_path, dtype, tol):
    """A mixer that caches one vector per position, registered from the test: the pools are
    allocated from its cache request (no keys, no values), beside an attention layer's group,
    and the model runs through every way of cutting with pages used again."""
    from rust_llm_inference_server_amd.engine import ModelRunner, load_model
    from rust_llm_inference_server_amd.registry import Architecture, register_architecture
    from rust_llm_inference_server_amd.weights import write_model_folder
    register_latent_toy()
    H, rank = 48, 20
    kinds = ["latent", "attention", "latent"]

    def build_spec(cfg):
        blocks = []
        for kind in cfg["mixers"]:
            if kind == "latent":
                blocks.append(layer_spec(H, 1, 1, 16, 64, 1e-5, 1e4, None, mixer="toy_latent_mean",
                                         extra={"hidden_size": H, "rank": rank}))
            else:
                blocks.append(layer_spec(H, 3, 1, 16, 64, 1e-5, 1e4, None))
        return toy_spec(blocks, H=H, V=cfg["vocab_size"])

    register_architecture(Architecture("ToyLatentForCausalLM", parse_config=lambda d: d,
                                       build_spec=build_spec, config_to_dict=lambda c: c))
    config = {"architectures": ["ToyLatentForCausalLM"], "vocab_size": 97, "mixers": kinds}
    folder = str(tmp_path / "latent")
    tdt = torch.float32 if dtype == "float32" else torch.bfloat16
    write_model_folder(folder, config, build_spec(config).tensor_specs(), seed=12, dtype=tdt)
    w = plain.read_weights(folder)

    def plain_model(ids):
        x = plain.embedding(w["model.embed_tokens.weight"], ids)
        for li, kind in enumerate(kinds):
            p = f"model.layers.{li}"
            h = plain.rms_norm(x, w[f"{p}.input_layernorm.weight"], 1e-5)
            if kind == "latent":
                lat = h @ w[f"{p}.self_attn.down.weight"].t()
                mean = lat.cumsum(0) / torch.arange(1, len(ids) + 1).unsqueeze(1)
                x = x + mean @ w[f"{p}.self_attn.up.weight"].t()
            else:
                cfg = {"num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 16}
                x = x + plain.attention_layer(h, w, f"{p}.self_attn", cfg, plain.inv_freqs(16, 1e4, None))
            h = plain.rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], 1e-5)
            x = x + plain.swiglu_mlp(h, w, f"{p}.mlp")
        return plain.linear(plain.rms_norm(x, w["model.norm.weight"], 1e-5), w["lm_head.weight"])

    reqs = traces.random_requests(97, [30, 4, 70, 11, 45, 2], seed=8)
    ref = {k: plain_model(t) for k, t in reqs.items()}
    for build in (traces.trace_whole, traces.trace_tail, traces.trace_portions, traces.trace_mixed):
        steps, max_tokens = build(reqs)
        model = load_model(folder, dtype, max_positions=128)
        assert len(model.cache_groups) == 2               # the latents' group and attention's
        latent_group = [g for g in model.cache_groups if g.request.arrays[0].name == "latent"][0]
        assert latent_group.request.elements_per_token() == rank and len(latent_group.writer_runs) == 2
        runner = ModelRunner(model, num_pages=max_tokens // 16, page_size=16, max_num_seqs=4)
        g = model.cache_groups.index(latent_group)
        assert set(runner.pools.arrays[g]) == {"latent"}
        assert runner.pools.arrays[g]["latent"].shape[2:] == (16, rank)
        # its pages are float32 in the bfloat16 model too, and are counted as such
        assert runner.pools.arrays[g]["latent"].dtype == torch.float32
        assert latent_group.request.bytes_per_token(model.act_dtype) == 4 * rank
        assert runner.pools.bytes_per_page(g) == 2 * 16 * rank * 4
        got = traces.collect(steps, traces.replay_in_process(runner, steps), 97)
        for k, tokens in reqs.items():
            mine = torch.stack([got[k][p] for p in range(len(tokens))])
            assert (mine - ref[k]).abs().max().item() < tol, f"{build.__name__} request {k}"
        for gi in range(runner.cache.num_groups):
            assert runner.cache.num_free_pages(gi) == runner.cache.num_pages(gi)


# ------------------------- a toy feed-forward with routing and a toy position encoding
def register_toy_router_and_position():
    """Both defined and registered here, in the test.  The feed-forward routes every row to
    the one expert whose router logit is largest (logits and their softmax in float32) and
    scales that expert's output by its probability; the position encoding is a rotation with
    frequencies of its own law over only a part of the head."""
    from rust_llm_inference_server_amd.parts import FeedForward, PositionEncoding, TensorSpec, register
    from rust_llm_inference_server_amd.parts.base import join

    @register("feed_forward", "toy_top1")
    class Top1Experts(FeedForward):
        @classmethod
        def tensor_specs(cls, params, prefix):
            H, I, E = params["hidden_size"], params["intermediate_size"], params["experts"]
            specs = [TensorSpec(join(prefix, "router.weight"), (E, H))]
            for e in range(E):
                specs += [TensorSpec(join(prefix, f"experts.{e}.up.weight"), (I, H)),
                          TensorSpec(join(prefix, f"experts.{e}.down.weight"), (H, I))]
            return specs

        def __init__(self, params, prefix, ctx):
            super().__init__(params, prefix, ctx)
            self.router = ctx.take(join(prefix, "router.weight")).float()
            self.up = [ctx.take(join(prefix, f"experts.{e}.up.weight")).float()
                       for e in range(params["experts"])]
            self.down = [ctx.take(join(prefix, f"experts.{e}.down.weight")).float()
                         for e in range(params["experts"])]
            self.act_dtype = ctx.act_dtype

        def forward(self, x, step):
            xf = x.float()
            prob = torch.softmax(xf @ self.router.t(), dim=-1)          # row by row
            top = prob.argmax(dim=-1)
            out = torch.zeros_like(xf)
            for e in range(len(self.up)):
                rows = (top == e).nonzero().reshape(-1)
                if rows.numel():
                    h = torch.relu(xf[rows] @ self.up[e].t())
                    out[rows] = (h @ self.down[e].t()) * prob[rows, e:e + 1]
            return out.to(self.act_dtype)

    @register("position", "toy_linear_frequencies")
    class LinearFrequencies(PositionEncoding):
        def __init__(self, params, prefix, ctx):
            super().__init__(params, prefix, ctx)
            self.rot_dim = int(params["rot_dim"])
            inv = (torch.arange(self.rot_dim // 2, dtype=torch.float32) + 1.0) * float(params["step"])
            angles = torch.arange(ctx.max_positions, dtype=torch.float32).reshape(-1, 1) * inv
            self.cos = torch.cos(angles).to(ctx.device).contiguous()
            self.sin = torch.sin(angles).to(ctx.device).contiguous()
            self.max_positions = ctx.max_positions


def plain_router_model(w, ids, H, nh, nkv, d, rot, step_size, experts, eps=1e-5, margins=None):
    """``margins`` (a list) receives every row's gap between its two largest router
    probabilities."""
    x = plain.embedding(w["model.embed_tokens.weight"], ids)
    T = len(ids)
    for li in range(2):
        p = f"model.layers.{li}"
        h = plain.rms_norm(x, w[f"{p}.input_layernorm.weight"], eps)
        if li == 0:       # rotation of the first `rot` dims only, with the toy frequencies
            inv = (torch.arange(rot // 2, dtype=torch.float32) + 1.0) * step_size
            cos, sin = plain.rope_tables(inv, range(T))
            q = plain.linear(h, w[f"{p}.self_attn.q_proj.weight"]).reshape(T, nh, d).transpose(0, 1)
            k = plain.linear(h, w[f"{p}.self_attn.k_proj.weight"]).reshape(T, nkv, d).transpose(0, 1)
            v = plain.linear(h, w[f"{p}.self_attn.v_proj.weight"]).reshape(T, nkv, d).transpose(0, 1)
            q = torch.cat([plain.rope_apply(q[..., :rot], cos, sin), q[..., rot:]], dim=-1)
            k = torch.cat([plain.rope_apply(k[..., :rot], cos, sin), k[..., rot:]], dim=-1)
            o = plain.gqa_attention(q, k, v, plain.causal_mask(T, 0, None))
            x = x + plain.linear(o.transpose(0, 1).reshape(T, nh * d), w[f"{p}.self_attn.o_proj.weight"])
            h = plain.rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], eps)
            prob = torch.softmax(plain.linear(h, w[f"{p}.mlp.router.weight"]), dim=-1)
            if margins is not None:
                top2 = prob.topk(2, dim=-1).values
                margins += (top2[:, 0] - top2[:, 1]).tolist()
            rows = []
            for t in range(T):
                e = int(prob[t].argmax())
                up = torch.relu(plain.linear(h[t:t + 1], w[f"{p}.mlp.experts.{e}.up.weight"]))
                rows.append(plain.linear(up, w[f"{p}.mlp.experts.{e}.down.weight"])[0] * prob[t, e])
            x = x + torch.stack(rows)
        else:
            cfg = {"num_attention_heads": nh, "num_key_value_heads": nkv, "head_dim": d}
            x = x + plain.attention_layer(h, w, f"{p}.self_attn", cfg, plain.inv_freqs(d, 1e4, None))
            h = plain.rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], eps)
            x = x + plain.swiglu_mlp(h, w, f"{p}.mlp")
    return plain.linear(plain.rms_norm(x, w["model.norm.weight"], eps), w["lm_head.weight"])


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-4), ("bfloat16", 4e-2)])
def test_toy_routed_feed_forward_and_toy_position_encoding(tmp_path, dtype, tol):
    """A feed-forward with routing and a position encoding, registered from the test, in one
    layer of a model whose other layer has the ordinary parts: built through the ordinary
    loader and replayed in every way of cutting."""
    from rust_llm_inference_server_amd.engine import ModelRunner, load_model
    from rust_llm_inference_server_amd.parts import PartSpec
    from rust_llm_inference_server_amd.registry import Architecture, register_architecture
    from rust_llm_inference_server_amd.weights import write_model_folder
    register_toy_router_and_position()
    H, nh, nkv, d, rot, E, I = 48, 3, 1, 32, 16, 3, 40

    def build_spec(cfg):
        first = layer_spec(H, nh, nkv, d, 64, 1e-5, 1e4, None)
        first.params["mixer"].params["position"] = PartSpec("toy_linear_frequencies",
                                                            {"rot_dim": rot, "step": cfg["step"]})
        first.params["feed_forward"] = PartSpec("toy_top1", {"hidden_size": H, "intermediate_size": I,
                                                             "experts": E})
        return toy_spec([first, layer_spec(H, nh, nkv, d, 64, 1e-5, 1e4, None)], H=H, V=cfg["vocab_size"])

    register_architecture(Architecture("ToyRoutedForCausalLM", parse_config=lambda c: c,
                                       build_spec=build_spec, config_to_dict=lambda c: c))
    config = {"architectures": ["ToyRoutedForCausalLM"], "vocab_size": 97, "step": 0.05}
    spec = build_spec(config)
    reqs = traces.random_requests(97, [30, 4, 70, 11], seed=10)
    # Weights for which no row's routing is a near-tie: a row whose two best experts are a hair
    # apart goes to either in bfloat16, and the other expert's output is another number
    # altogether.  The first seed whose closest call is clear of that is taken.
    for seed in range(12, 60):
        folder = str(tmp_path / f"toy_routed_{seed}")
        write_model_folder(folder, config, spec.tensor_specs(), seed=seed)
        w = plain.read_weights(folder)
        margins = []
        ref = {k: plain_router_model(w, t, H, nh, nkv, d, rot, 0.05, E, margins=margins)
               for k, t in reqs.items()}
        if min(margins) > 2e-3:
            break
    assert min(margins) > 2e-3, "no seed gave clear routing"
    for build in (traces.trace_whole, traces.trace_tail, traces.trace_portions, traces.trace_mixed):
        steps, max_tokens = build(reqs)
        model = load_model(folder, dtype, max_positions=128)
        # the toy feed-forward decides on the host: this model's decode steps are not captured
        assert not model.graph_safe
        runner = ModelRunner(model, num_pages=max_tokens // 16, page_size=16, max_num_seqs=4)
        got = traces.collect(steps, traces.replay_in_process(runner, steps), 97)
        for k, tokens in reqs.items():
            mine = torch.stack([got[k][p] for p in range(len(tokens))])
            diff = (mine - ref[k]).abs().max(dim=-1).values
            assert diff.max().item() < tol, (f"{build.__name__} request {k}: first wrong position "
                                             f"{int((diff >= tol).nonzero()[0])}")
    # the routing really spreads the rows over the experts
    h = plain.rms_norm(plain.embedding(w["model.embed_tokens.weight"], reqs["r2"]),
                       w["model.layers.0.input_layernorm.weight"], 1e-5)
    used = set(torch.softmax(plain.linear(h, w["model.layers.0.mlp.router.weight"]), -1).argmax(-1).tolist())
    assert len(used) >= 2


def register_toy_biased_position():
    """Defined and registered here, in the test: a position encoding that does both things the
    built-in one does not: its rotation pairs neighbouring dims (2j with 2j + 1) over a part of
    the head, and it adds slope * (key position - query position) to every score."""
    from rust_llm_inference_server_amd.parts import PositionEncoding, register

    @register("position", "toy_interleaved_with_bias")
    class InterleavedWithBias(PositionEncoding):
        def __init__(self, params, prefix, ctx):
            super().__init__(params, prefix, ctx)
            self.rot_dim = int(params["rot_dim"])
            self.interleaved = True
            inv = plain.inv_freqs(self.rot_dim, float(params["theta"]), None)
            angles = torch.arange(ctx.max_positions, dtype=torch.float32).reshape(-1, 1) * inv
            self.cos = torch.cos(angles).to(ctx.device).contiguous()
            self.sin = torch.sin(angles).to(ctx.device).contiguous()
            self.bias_slopes = torch.tensor(params["slopes"], dtype=torch.float32, device=ctx.device)
            self.max_positions = ctx.max_positions

    return InterleavedWithBias


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-4), ("bfloat16", 4e-2)])
def test_toy_position_encoding_with_another_layout_and_a_score_bias(tmp_path, dtype, tol):
    """The attention mixer with a position part, registered from the test, that rotates
    neighbouring dims over half of the head and biases the scores by distance: the first layer
    of a model whose second layer is the ordinary one, through every way of cutting.  The bias
    is strong enough that leaving it out would show."""
    from rust_llm_inference_server_amd.engine import ModelRunner, load_model
    from rust_llm_inference_server_amd.parts import PartSpec
    from rust_llm_inference_server_amd.registry import Architecture, register_architecture
    from rust_llm_inference_server_amd.weights import write_model_folder
    register_toy_biased_position()
    H, nh, nkv, d, rot = 48, 4, 2, 32, 16
    slopes = [0.5, 0.25, 0.125, 0.0625]

    def build_spec(cfg):
        first = layer_spec(H, nh, nkv, d, 64, 1e-5, 1e4, None)
        first.params["mixer"].params["position"] = PartSpec(
            "toy_interleaved_with_bias", {"rot_dim": rot, "theta": 1e4, "slopes": cfg["slopes"]})
        return toy_spec([first, layer_spec(H, nh, nkv, d, 64, 1e-5, 1e4, None)], H=H, V=cfg["vocab_size"])

    register_architecture(Architecture("ToyBiasedForCausalLM", parse_config=lambda c: c,
                                       build_spec=build_spec, config_to_dict=lambda c: c))
    config = {"architectures": ["ToyBiasedForCausalLM"], "vocab_size": 97, "slopes": slopes}
    folder = str(tmp_path / "toy_biased")
    tdt = torch.float32 if dtype == "float32" else torch.bfloat16
    write_model_folder(folder, config, build_spec(config).tensor_specs(), seed=14, dtype=tdt)
    w = plain.read_weights(folder)

    def plain_model(ids, with_bias=True):
        x = plain.embedding(w["model.embed_tokens.weight"], ids)
        T = len(ids)
        for li in range(2):
            p = f"model.layers.{li}"
            h = plain.rms_norm(x, w[f"{p}.input_layernorm.weight"], 1e-5)
            if li == 0:
                inv = plain.inv_freqs(rot, 1e4, None)
                cos, sin = plain.rope_tables(inv, range(T))

                def rotate(t):                      # (heads, T, d): pairs (2j, 2j + 1) below rot
                    out = t.clone()
                    a, b = t[..., 0:rot:2], t[..., 1:rot:2]
                    out[..., 0:rot:2] = a * cos - b * sin
                    out[..., 1:rot:2] = b * cos + a * sin
                    return out

                q = rotate(plain.linear(h, w[f"{p}.self_attn.q_proj.weight"]).reshape(T, nh, d).transpose(0, 1))
                k = rotate(plain.linear(h, w[f"{p}.self_attn.k_proj.weight"]).reshape(T, nkv, d).transpose(0, 1))
                v = plain.linear(h, w[f"{p}.self_attn.v_proj.weight"]).reshape(T, nkv, d).transpose(0, 1)
                dist = (torch.arange(T).reshape(1, -1) - torch.arange(T).reshape(-1, 1)).float()
                heads = []
                for hh in range(nh):
                    mask = plain.causal_mask(T, 0, None) + (slopes[hh] * dist if with_bias else 0.0)
                    kv = hh // (nh // nkv)
                    heads.append(plain.gqa_attention(q[hh:hh + 1], k[kv:kv + 1], v[kv:kv + 1], mask)[0])
                o = torch.stack(heads)
                x = x + plain.linear(o.transpose(0, 1).reshape(T, nh * d), w[f"{p}.self_attn.o_proj.weight"])
            else:
                cfg = {"num_attention_heads": nh, "num_key_value_heads": nkv, "head_dim": d}
                x = x + plain.attention_layer(h, w, f"{p}.self_attn", cfg, plain.inv_freqs(d, 1e4, None))
            h = plain.rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], 1e-5)
            x = x + plain.swiglu_mlp(h, w, f"{p}.mlp")
        return plain.linear(plain.rms_norm(x, w["model.norm.weight"], 1e-5), w["lm_head.weight"])

    reqs = traces.random_requests(97, [30, 4, 70, 11], seed=10)
    ref = {k: plain_model(t) for k, t in reqs.items()}
    assert (ref["r2"] - plain_model(reqs["r2"], with_bias=False)).abs().max().item() > 4 * tol
    for build in (traces.trace_whole, traces.trace_tail, traces.trace_portions, traces.trace_mixed):
        steps, max_tokens = build(reqs)
        model = load_model(folder, dtype, max_positions=128)
        runner = ModelRunner(model, num_pages=max_tokens // 16, page_size=16, max_num_seqs=4)
        got = traces.collect(steps, traces.replay_in_process(runner, steps), 97)
        for k, tokens in reqs.items():
            mine = torch.stack([got[k][p] for p in range(len(tokens))])
            diff = (mine - ref[k]).abs().max(dim=-1).values
            assert diff.max().item() < tol, (f"{build.__name__} request {k}: first wrong position "
                                             f"{int((diff >= tol).nonzero()[0])}")


def test_long_decoding_stays_on_the_plain_path(tiny_folders):
    """A short prompt, then 230 tokens one by one (teacher-forced), across many page edges."""
    from rust_llm_inference_server_amd.engine import ModelRunner, StepEntry, load_model
    folder = tiny_folders["b"]
    w, c = plain.read_weights(folder), plain.read_config(folder)
    ids = traces.random_requests(c["vocab_size"], [240], seed=12)["r0"]
    ref = plain.forward(w, c, ids)
    for dtype, tol in (("float32", 1e-4), ("bfloat16", 3e-2)):
        model = load_model(folder, dtype, max_positions=256)
        runner = ModelRunner(model, num_pages=32, page_size=8, max_num_seqs=2)
        runner.reserve(0, 10)
        rows = [runner.step([StepEntry(0, ids[:10], list(range(10)))]).cpu()]
        for p in range(10, len(ids)):
            runner.reserve(0, p + 1)
            rows.append(runner.step([StepEntry(0, [ids[p]], [0])]).cpu())
        diff = (torch.cat(rows) - ref).abs().max(dim=-1).values
        assert diff.max().item() < tol, f"{dtype}: first wrong position {int((diff >= tol).nonzero()[0])}"
