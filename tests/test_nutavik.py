"""Nutavik in the engine against the plain implementation (tests/plain_nutavik.py): every way of
cutting the work, on the CPU with plain PyTorch ops (the host side: batching, paging, slots, the
order of parts) and, marked ``gpu``, with the HIP kernels in true float32 and in bfloat16."""
import copy
import json
import os

import pytest
import torch

import nutavik_cases as X
import plain_nutavik as P
import replay_cases as C
from kernel_refs import RefOps

BACKENDS = [
    pytest.param(("cpu", "float32"), id="cpu-ref-f32"),
    pytest.param(("cuda:0", "float32"), id="hip-f32", marks=pytest.mark.gpu),
    pytest.param(("cuda:0", "bfloat16"), id="hip-bf16", marks=pytest.mark.gpu),
]
_ops = {}
_plain = {}


def ops_for(device):
    if device == "cpu":
        return RefOps()
    if device not in _ops:
        from yalis_amd.ops.hip import HipOps

        _ops[device] = HipOps(device)
    return _ops[device]


def setup(name):
    cfg = X.CONFIGS[name]
    if name not in _plain:
        weights = X.random_weights(cfg, seed=len(name))
        reqs = X.make_requests(cfg, X.LENGTHS[name], seed=10)
        _plain[name] = (weights, reqs, X.plain_logits(cfg, weights, reqs))
    return (cfg, *_plain[name])


TRACES = {"whole": C.trace_whole, "tail": C.trace_tail, "one_by_one": lambda r: C.trace_tail(r, tail=1 << 20),
          "portions": C.trace_portions, "mixed": C.trace_mixed, "random": lambda r: C.trace_random(r, 5)}


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["odd", "mix", "wide"])
@pytest.mark.parametrize("mode", list(TRACES))
def test_replay_modes(backend, name, mode):
    """Whole prompts; a prompt and then its last tokens one by one; every token one by one (prefill
    against decoding); portions down to two tokens; up to four unequal requests a step in a pool so
    small that pages and slots are used again; cuts at random."""
    device, dtype = backend
    if device == "cpu" and (name == "wide" or (name == "mix" and mode not in ("whole", "mixed", "portions"))):
        pytest.skip("the plain ops are slow at this size; the GPU runs every mode")
    cfg, weights, reqs, want = setup(name)
    steps = TRACES[mode](reqs)
    page = X.PAGE[name]
    n_pages = C.pages_needed(steps, reqs, page)
    runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), page, n_pages)
    got, rp = C.run_trace(runner, steps)
    X.assert_matches(got, want, dtype == "bfloat16", f"{name}/{mode}")
    runner.pages.audit()
    assert runner.pages.live_requests() == 0
    assert all(runner.pages.free_pages(g) == n_pages for g in range(len(runner.group_shapes)))
    if mode == "mixed":
        owners, reused = {}, False
        for held in rp.page_log:
            for rid, tables in held.items():
                for g, pages in enumerate(tables):
                    for p in pages:
                        if p >= 0:
                            reused |= owners.setdefault((g, p), rid) != rid
        assert reused, "the trace was meant to reuse pages"


def test_memory_plan():
    """Caches group by the length of their rows; a layer that reads another's cache owns none; the
    recurrent layers keep a matrix per head and, with more than one tap, the convolution's inputs."""
    cfg, weights, _, _ = setup("mix")
    runner = X.make_runner(cfg, weights, "float32", "cpu", RefOps(), 32, 4)
    m = runner.model
    assert [(g.need.num_kv_heads, g.need.head_dim, g.need.v_dim, len(g.entries)) for g in m.cache_groups] == [(1, 32, 0, 1), (1, 64, 0, 1)]
    assert [s.owns_cache for s in m.sites] == [False, True, False, True, False, False, False]
    assert (m.sites[4].group, m.sites[6].group) == (m.sites[1].group, m.sites[3].group)
    assert [tuple(s.shape) for s in m.state_needs] == [(4, 16, 16), (2, 32, 48), (1, 2 * 2 * 32 + 2 * 48), (8, 8, 8)]
    assert all(v is None for v in runner.memory.values), "a page row serves as key and value: no value pages"


@pytest.mark.parametrize("backend", BACKENDS)
def test_slots_are_used_again_with_clean_state(backend):
    """Two slots, five requests one after another in pairs: a request that takes over a slot starts
    from a zero matrix and an empty convolution, whatever the one before left there."""
    device, dtype = backend
    cfg, weights, reqs, want = setup("odd")
    runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 16, max_seqs=2)
    steps = C.trace_mixed(reqs, max_live=2)
    got, _ = C.run_trace(runner, steps)
    X.assert_matches(got, want, dtype == "bfloat16", "two slots")
    assert runner.pages.free_slots() == 2


@pytest.mark.parametrize("backend", BACKENDS)
def test_long_decoding(backend):
    """A short prompt and 200 tokens decoded one by one: the states are carried through every step,
    the attention reads pages written by hundreds of earlier steps."""
    device, dtype = backend
    cfg = X.CONFIGS["odd"]
    weights = X.random_weights(cfg, seed=21)
    reqs = X.make_requests(cfg, [215], seed=3)
    want = X.plain_logits(cfg, weights, reqs)
    runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 14, max_seqs=1)
    got, _ = C.run_trace(runner, C.trace_tail(reqs, tail=200))
    X.assert_matches(got, want, dtype == "bfloat16", "long decoding")


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["mix", "wide"])
def test_long_prompt_in_one_step(backend, name):
    """A prompt of 450 tokens whole, then a few tokens one by one; and the same prompt in portions
    whose edges fall inside pages and inside the blocks of keys the attention walks."""
    device, dtype = backend
    if device == "cpu":
        pytest.skip("the plain ops are slow at this size; the GPU runs it")
    cfg = X.CONFIGS[name]
    weights = X.random_weights(cfg, seed=31)
    reqs = X.make_requests(cfg, [456], seed=8)
    want = X.plain_logits(cfg, weights, reqs)
    runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), X.PAGE[name], 16, max_seqs=1)
    got, _ = C.run_trace(runner, C.trace_tail(reqs, tail=6))
    X.assert_matches(got, want, dtype == "bfloat16", f"{name}/long prompt")
    runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), X.PAGE[name], 16, max_seqs=1)
    got, _ = C.run_trace(runner, C.trace_portions(reqs, sizes=[70, 2, 33, 64, 5, 100]))
    X.assert_matches(got, want, dtype == "bfloat16", f"{name}/long prompt in portions")


def _one_layer(layer, ff, mult=0.7, logit_scale=1.5):
    return X.model(80, 32, 1e-5, mult, logit_scale, [(layer, ff)])


MECHANISMS = {
    "latent_attention": _one_layer(X.latent(2, 8, 4, 8, 12, 16, 10.0, 0.4), None),
    "latent_attention_scaled_rotation": _one_layer(X.latent(3, 4, 16, 6, 8, 8, 10.0, 0.2, scaling=X.YARN_A), None),
    "delta": _one_layer(X.delta(2, 2, 8, 8, 4), None),
    "delta_shared_keys_one_tap": _one_layer(X.delta(6, 2, 16, 4, 1), None),
    "delta_wide_keys": _one_layer(X.delta(1, 1, 40, 3, 2), None),
    "gla": _one_layer(X.gla(2, 8, 8, 2.0, low_rank=3), None),
    "gla_tau_one": _one_layer(X.gla(3, 24, 5, 1.0), None),
    "dense": _one_layer(X.gla(1, 8, 8, 8.0, low_rank=2), 48),
}


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("which", list(MECHANISMS))
def test_each_mechanism_alone(backend, which):
    """One-layer models, each with one mechanism, whole and in portions; on the CPU the residual
    stream after the layer is compared too (a wrong multiplier could hide behind the final norm)."""
    device, dtype = backend
    cfg = MECHANISMS[which]
    weights = X.random_weights(cfg, seed=5)
    reqs = X.make_requests(cfg, [37, 12], seed=1)
    want = X.plain_logits(cfg, weights, reqs)
    for make in (C.trace_whole, C.trace_portions):
        runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 8)
        got, _ = C.run_trace(runner, make(reqs))
        X.assert_matches(got, want, dtype == "bfloat16", which)


@pytest.mark.parametrize("backend", BACKENDS)
def test_residual_stream_after_every_layer(backend):
    """The float32 stream the engine holds after its last layer equals the plain one (the pending
    branch added): multiplier, both norms of each branch and their biases all show here."""
    device, dtype = backend
    cfg, weights, reqs, _ = setup("odd")
    toks = reqs["r2"]
    streams = []
    P.forward(cfg, weights, torch.tensor(toks), streams)
    for depth in range(1, len(cfg["layers"]) + 1):
        cut = copy.deepcopy(cfg)
        cut["layers"] = cut["layers"][:depth]
        names = X.tensor_specs_for(cut)
        runner = X.make_runner(cut, {k: weights[k] for k in names}, dtype, device, ops_for(device), 16, 8)
        captured = {}
        final = runner.model.final_norm
        original = final.gather_add_norm

        def spy(residual, delta, rows, _original=original):
            out = _original(residual, delta, rows)
            settled = residual.clone()
            if delta is not None:
                delta.settle(settled)
            captured["x"] = settled.float().cpu()
            return out

        final.gather_add_norm = spy
        C.run_trace(runner, C.trace_whole({"a": toks}))
        want = streams[depth - 1]
        err = (captured["x"].double() - want).abs().max().item() / want.abs().max().item()
        assert err < (3e-2 if dtype == "bfloat16" else 1e-5), f"stream after layer {depth - 1}: relative error {err:.2e}"


@pytest.mark.parametrize("backend", BACKENDS)
def test_sharp_attention_over_a_long_prompt(backend):
    """Scores multiplied so hard that nearly every query gives most of its weight to one key, which lies
    anywhere among the 300 before it: a key lost or misplaced at a page's border, at the border of a
    block of keys, among the first tokens or hundreds of tokens back changes that query's logits
    outright instead of by a three-hundredth.  (tests/test_nutavik_kernels_gpu.py places one such key at
    every border by hand.)"""
    device, dtype = backend
    cfg = _one_layer(X.latent(2, 8, 4, 8, 12, 16, 10.0, 6.0), None)
    weights = X.random_weights(cfg, seed=13)
    toks = X.make_requests(cfg, [300], seed=2)["r0"]
    want = {"a": P.forward(cfg, weights, torch.tensor(toks))}
    # how sharp: the plain attention's largest weight per query and head
    W = {k: v.double() for k, v in weights.items()}
    h = P.layer_norm(W["embed"][torch.tensor(toks)], W["l0.norm1"], W["l0.norm1.b"], 1e-5)
    m = cfg["layers"][0]["mixer"]
    soft = dict(m, scale=m["scale"])
    latents = {}
    P.latent_attention(W, "l0.mix.", soft, 1e-5, h, latents, 0)
    c, kt = latents[0]
    c_q = P.rms_norm(h @ W["l0.mix.dq"].T, W["l0.mix.dq.norm"], 1e-5)
    q = (c_q @ W["l0.mix.uq"].T).view(300, 2, 12)
    cos, sin = P.rotation_tables(m["rot"], 300)
    k = (c @ W["l0.mix.uk"].T).view(300, 2, 8)
    sc = (torch.einsum("ihd,jhd->hij", q[..., :8], k) + torch.einsum("ihd,jd->hij", P.turn_pairs(q[..., 8:], cos, sin), kt)) * m["scale"]
    sc = sc.masked_fill(~torch.tril(torch.ones(300, 300, dtype=torch.bool)), float("-inf"))
    peak = torch.softmax(sc, -1).max(-1)
    assert peak.values[:, 100:].median().item() > 0.5, "the test's attention was meant to be sharp"
    assert (peak.indices[:, 200:] < 100).any(), "some late query was meant to pick a key far back"
    for make in (lambda r: C.trace_tail(r, tail=40), C.trace_portions):
        runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 24, max_len=512)
        got, _ = C.run_trace(runner, make({"a": toks}))
        X.assert_matches(got, want, dtype == "bfloat16", "sharp attention")


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("num_pages", [24, 7])
def test_greedy_generation_through_the_engine(tmp_path, backend, num_pages):
    """``LLMEngine.generate`` with the scheduler under a token budget that cuts prompts into
    portions, and with so few pages that the youngest request is preempted and starts again (its
    state slot cleared): greedy tokens are the plain implementation's wherever its two best logits
    are clearly apart."""
    from yalis_amd import EngineConfig, InferenceConfig, LLMEngine, ModelConfig
    from yalis_amd.weights.safetensors_io import write_dict

    device, dtype = backend
    cfg = X.CONFIGS["odd"]
    weights = X.random_weights(cfg, seed=9)
    folder = tmp_path / "model"
    os.makedirs(folder)
    with open(folder / "config.json", "w") as f:
        json.dump(cfg, f)
    wd = torch.float32 if dtype == "float32" else torch.bfloat16
    write_dict(str(folder / "model.safetensors"), {k: v.to(wd).contiguous() for k, v in weights.items()})
    precision = "fp32" if dtype == "float32" else "bf16"
    eng = LLMEngine(
        ModelConfig(model_path=str(folder), precision=precision),
        InferenceConfig(max_batch_size=3, max_length_of_generated_sequences=128, temperature=0.0),
        device=device, ops=RefOps() if device == "cpu" else None,
        engine_config=EngineConfig(page_size=16, num_pages=num_pages, max_num_seqs=3, max_model_len=128, max_num_batched_tokens=24,
                                   dtype=dtype, device=device),
    )
    prompts = list(X.make_requests(cfg, [30, 7, 45], seed=4).values())
    out, metrics = eng.generate(prompts, tokens_to_generate=12)
    assert out.shape == (3, 12)
    if num_pages == 7:
        assert metrics["Preemptions"] > 0, "this pool was meant to force a preemption"
    gap = 0.2 if dtype == "bfloat16" else 1e-3
    for prompt, row in zip(prompts, out.tolist()):
        toks = list(prompt)
        for t in row:
            logits = P.forward(cfg, weights, torch.tensor(toks))[-1]
            top2 = torch.topk(logits, 2).values
            if (top2[0] - top2[1]).item() < gap * logits.abs().max().item():
                break  # too close to call; what follows would compare other sequences
            assert t == int(torch.argmax(logits)), f"generated {row}, the plain implementation differs after {len(toks) - len(prompt)} tokens"
            toks.append(t)


def test_config_reader_and_spec():
    """Sizes and constants come from config.json; what cannot run is refused with the key's name; the
    tensors a model asks for are the design's names and shapes; a layer that reads another's cache
    becomes a run entry that borrows it and asks for no down-projection of its own."""
    from yalis_amd.config.reader import ConfigError
    from yalis_amd.engine.factory import spec_from_config, tensor_specs_for

    cfg = X.CONFIGS["mix"]
    _, typed, spec = spec_from_config(cfg)
    assert spec.vocab_size == 128 and spec.hidden_size == 64 and len(spec.layers) == 7
    assert spec.head.params["tied_to"] == "embed" and spec.head.params["scale"] == 3.0
    assert all(layer.block == "sandwich" and layer.params["branch_scale"] == 0.5 for layer in spec.layers)
    att = spec.layers[1].parts["mixer"].params
    assert (att["num_heads"], att["head_dim"], att["rot_dim"], att["value_dim"], att["kv_rank"], att["q_rank"]) == (2, 32, 8, 16, 24, 40)
    assert att["position"].params["scaling"]["kind"] == "yarn" and att["position"].params["pairing"] == "interleaved"
    assert [e.cache_from for e in spec.run_order] == [None, None, None, None, 1, None, 3]
    assert "feed_forward" not in spec.layers[2].parts and "feed_forward_out_norm" in spec.layers[0].parts
    assert spec.layers[5].parts["mixer"].kind == "delta_rule" and spec.layers[5].parts["mixer"].params["conv_taps"] == 1
    specs = tensor_specs_for(cfg)
    assert specs["l1.mix.dkv"].shape == (32, 64) and specs["l1.mix.uq"].shape == (2 * 40, 40) and specs["l1.mix.g"].shape == (2, 64)
    assert "l4.mix.dkv" not in specs and "l4.mix.dkv.norm" not in specs and specs["l4.mix.uk"].shape == (4 * 16, 24)
    assert specs["l2.mix.k.conv"].shape == (64, 2) and specs["l2.mix.v"].shape == (96, 64) and specs["l5.mix.A_log"].shape == (8,)
    assert specs["l0.mix.a2.b"].shape == (64,) and specs["l0.mix.norm"].shape == (16,) and specs["l0.norm1b.b"].shape == (64,)
    assert "l2.norm2" not in specs and specs["final.norm.b"].shape == (64,) and "head" not in specs
    for path, value, what in [
        (("layers", 2, "mixer", "kv_heads"), 3, "multiple"), (("layers", 1, "mixer", "rot", "dims"), 6, "rot_dim"),
        (("layers", 0, "type"), "attention", "not one of"), (("layers", 4, "mixer", "kv_from"), 2, "earlier latent_attention"),
        (("layers", 4, "mixer", "kv_from"), 5, "earlier latent_attention"), (("layers", 6, "mixer", "kv_from"), 4, "of its own"),
        (("layers", 4, "mixer", "kv_rank"), 32, "differs"), (("layers", 0, "mlp", "kind"), "moe", "not supported"),
    ]:
        bad = copy.deepcopy(cfg)
        node = bad
        for key in path[:-1]:
            node = node[key]
        node[path[-1]] = value
        with pytest.raises(ConfigError, match=what):
            spec_from_config(bad)
    missing = copy.deepcopy(cfg)
    del missing["layers"][1]["mixer"]["scale"]
    with pytest.raises(ConfigError, match="scale"):
        spec_from_config(missing)


def test_decay_rank_comes_from_the_checkpoint(tmp_path):
    """Nothing in config.json says how narrow the decay's pair of projections is: a folder whose
    tensors have another rank than the random-weights mode would make loads, and one whose two
    tensors disagree is refused."""
    from yalis_amd.config.runtime import EngineConfig
    from yalis_amd.engine.factory import load_runner
    from yalis_amd.weights.safetensors_io import write_dict

    cfg = _one_layer(X.gla(2, 8, 8, 2.0), None)
    weights = X.random_weights(cfg, seed=3)
    g = torch.Generator().manual_seed(1)
    weights["l0.mix.a1"] = (torch.randn((7, 32), generator=g) * 0.3).to(torch.bfloat16).float()
    weights["l0.mix.a2"] = (torch.randn((16, 7), generator=g) * 0.3).to(torch.bfloat16).float()
    folder = tmp_path / "model"
    os.makedirs(folder)
    with open(folder / "config.json", "w") as f:
        json.dump(cfg, f)
    write_dict(str(folder / "model.safetensors"), {k: v.contiguous() for k, v in weights.items()})
    eng = EngineConfig(page_size=16, num_pages=4, max_num_seqs=2, max_model_len=64, max_num_batched_tokens=64, dtype="float32", device="cpu")
    runner = load_runner(str(folder), eng, ops=RefOps())
    toks = X.make_requests(cfg, [20], seed=1)
    got, _ = C.run_trace(runner, C.trace_whole(toks))
    X.assert_matches(got, X.plain_logits(cfg, weights, toks), False, "rank 7")
    weights["l0.mix.a2"] = weights["l0.mix.a2"][:, :6].contiguous()
    write_dict(str(folder / "model.safetensors"), {k: v.contiguous() for k, v in weights.items()})
    with pytest.raises(ValueError, match="rank"):
        load_runner(str(folder), eng, ops=RefOps())
