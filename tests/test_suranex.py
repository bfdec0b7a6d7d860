"""Suranex in the engine against the plain implementation (tests/plain_suranex.py): every way of
cutting the work, on the CPU with plain PyTorch ops (the host side: batching, paging, slots, the
order of parts) and, marked ``gpu``, with the HIP kernels in true float32 and in bfloat16."""
import json
import os

import pytest
import torch

import plain_suranex as S
import replay_cases as C
import suranex_cases as X
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
    if device == "cpu" and name == "wide" and mode not in ("whole", "mixed"):
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


@pytest.mark.parametrize("backend", BACKENDS)
def test_slots_are_used_again_with_clean_state(backend):
    """Two slots, five requests one after another in pairs: a request that takes over a slot starts
    from a zero state, whatever the one before left there."""
    device, dtype = backend
    cfg, weights, reqs, want = setup("mix")
    runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 32, 16, max_seqs=2)
    steps = C.trace_mixed(reqs, max_live=2)
    got, _ = C.run_trace(runner, steps)
    X.assert_matches(got, want, dtype == "bfloat16", "two slots")
    assert runner.pages.free_slots() == 2


@pytest.mark.parametrize("backend", BACKENDS)
def test_long_decoding(backend):
    """A short prompt and 220 tokens decoded one by one: the window passes over decoded tokens
    several times, kept first keys stay, the recurrent state is carried through every step, and
    pages that fell out of the window were given back on the way."""
    device, dtype = backend
    cfg = X.CONFIGS["mix"]
    weights = X.random_weights(cfg, seed=21)
    reqs = X.make_requests(cfg, [240], seed=3)
    want = X.plain_logits(cfg, weights, reqs)
    runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), 16, 20, max_seqs=1)
    steps = C.trace_tail(reqs, tail=220)
    got, rp = C.run_trace(runner, steps)
    X.assert_matches(got, want, dtype == "bfloat16", "long decoding")
    # the layer with a window of 20 keys and 5 kept first ones holds its first page and the last few only
    windowed = [g for g, s in enumerate(runner.group_shapes) if s.window == 20]
    held = rp.page_log[-2]["r0"][windowed[0]]
    assert held[0] >= 0 and held[1] < 0 and held[-1] >= 0 and sum(p >= 0 for p in held) <= 4


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["mix", "wide"])
def test_long_prompt_in_one_step(backend, name):
    """A prompt of 450 tokens whole, then a few tokens one by one: a span of many scan chunks, experts
    with more than a hundred pairs each (the largest tiles), attention tiles far from the start."""
    device, dtype = backend
    if device == "cpu" and name == "wide":
        pytest.skip("the plain ops are slow at this size; the GPU runs it")
    cfg = X.CONFIGS[name]
    weights = X.random_weights(cfg, seed=31)
    reqs = X.make_requests(cfg, [456], seed=8)
    want = X.plain_logits(cfg, weights, reqs)
    runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), X.PAGE[name], 16, max_seqs=1)
    got, _ = C.run_trace(runner, C.trace_tail(reqs, tail=6))
    X.assert_matches(got, want, dtype == "bfloat16", f"{name}/long prompt")
    # the same prompt in portions: the windows give pages back on the way, and later portions read
    # kept first keys from pages that stayed beside keys whose pages are gone
    runner = X.make_runner(cfg, weights, dtype, device, ops_for(device), X.PAGE[name], 16, max_seqs=1)
    got, rp = C.run_trace(runner, C.trace_portions(reqs, sizes=[70, 2, 33, 64, 5, 100]))
    X.assert_matches(got, want, dtype == "bfloat16", f"{name}/long prompt in portions")
    assert any(p < 0 for tables in rp.page_log[-2]["r0"] for p in tables), "some window was meant to give pages back"


def _one_layer(layer, mlp):
    return X.model(80, 32, 1e-5, [(layer, mlp)])


MECHANISMS = {
    "recurrence": _one_layer(X.rglru(48, 3, 4), None),
    "recurrence_one_tap": _one_layer(X.rglru(32, 2, 1), None),
    "attention_window_and_first": _one_layer(X.attention(2, 1, 16, 16, 7, 2, 16, 10.0, 0.4), None),
    "attention_partial_rotation_scaled": _one_layer(X.attention(2, 2, 32, 16, None, 0, 8, 10.0, 0.2, scaling=X.YARN_A), None),
    "attention_squashed": _one_layer(X.attention(4, 2, 16, 32, 11, 0, 16, 10.0, 2.0, softcap=1.5), None),
    "experts": _one_layer(X.rglru(32, 1, 2), X.moe(5, 2, 16, 0.5)),
    "experts_and_shared": _one_layer(X.rglru(32, 1, 2), X.moe(3, 1, 24, 1.0, shared=(8, 0.25))),
}


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("which", list(MECHANISMS))
def test_each_mechanism_alone(backend, which):
    """One-layer models, each with one mechanism; the residual stream after the layer is compared
    too (through the logits of an identity-like head it would hide behind the final norm)."""
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
    write_dict(str(folder / "model.safetensors"), {k: (v if v.dtype == torch.int32 else v.to(wd)).contiguous() for k, v in weights.items()})
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
            logits = S.forward(cfg, weights, torch.tensor(toks))[-1]
            top2 = torch.topk(logits, 2).values
            if (top2[0] - top2[1]).item() < gap * logits.abs().max().item():
                break  # too close to call; what follows would compare other sequences
            assert t == int(torch.argmax(logits)), f"generated {row}, the plain implementation differs after {len(toks) - len(prompt)} tokens"
            toks.append(t)


def test_config_reader_and_spec():
    """Sizes and constants come from config.json; what cannot run is refused with the key's name; the
    tensors a model asks for are the design's names and shapes."""
    import copy

    from yalis_amd.config.reader import ConfigError
    from yalis_amd.engine.factory import spec_from_config, tensor_specs_for

    cfg = X.CONFIGS["mix"]
    _, typed, spec = spec_from_config(cfg)
    assert spec.vocab_size == 128 and spec.hidden_size == 64 and len(spec.layers) == 5
    att = spec.layers[1].parts["mixer"].params
    assert (att["window"], att["keep_first"], att["softcap"], att["value_dim"], att["head_dim"]) == (20, 5, 30.0, 32, 32)
    assert att["position"].params["scaling"]["kind"] == "yarn" and att["position"].params["rotary_dim"] == 16
    assert spec.layers[2].parts["mixer"].params["window"] is None, "no mask: every earlier key"
    assert "feed_forward" not in spec.layers[2].parts and "feed_forward" in spec.layers[0].parts
    assert spec.layers[4].parts["mixer"].kind == "rglru" and spec.layers[4].parts["mixer"].params["conv_taps"] == 5
    specs = tensor_specs_for(cfg)
    assert specs["l0.mix.ra"].shape == (1, 64, 64) and specs["l0.mix.conv"].shape == (64, 2) and specs["l0.mlp.table"].shape == (128, 3)
    assert specs["l1.mix.g"].shape == (4, 64) and specs["l1.mix.q.norm"].shape == (32,) and specs["l2.mix.o"].shape == (64, 2 * 64)
    assert specs["l0.mlp.shared.gate"].shape == (64, 64) and "l1.mlp.shared.gate" not in specs and "l2.norm2" not in specs
    for path, value, what in [
        (("layers", 1, "mixer", "kv_heads"), 3, "multiple"), (("layers", 1, "mixer", "vdim"), 7, "even"),
        (("layers", 1, "mixer", "rot", "dims"), 40, "at most"), (("layers", 0, "type"), "conv", "not one of"),
        (("layers", 0, "mixer", "blocks"), 5, "divide"), (("layers", 0, "mlp", "router", "top"), 9, "top"),
        (("layers", 0, "mlp", "kind"), "dense", "not supported"),
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
