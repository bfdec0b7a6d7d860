"""Small Suranex configurations that differ from each other in every size and option, random
weights for them, and helpers to run them through the engine and the plain implementation."""
from __future__ import annotations

import copy
from typing import Dict, List, Sequence

import torch

import plain_suranex as S
from yalis_amd.config.runtime import EngineConfig
from yalis_amd.engine.factory import build_model, tensor_specs_for
from yalis_amd.engine.step import ModelRunner


def attention(heads, kv, dim, vdim, size, keep, dims, base, scale, softcap=None, scaling=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "softcap": softcap,
         "rot": {"base": base, "dims": dims, "scaling": scaling}}
    if size is not None:
        m["mask"] = {"size": size, "keep_first": keep}
    return {"type": "attention", "mixer": m}


def rglru(width, blocks, conv):
    return {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": conv}}


def moe(experts, top, ff, limit, shared=None):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit},
            "shared": None if shared is None else {"ff": shared[0], "limit": shared[1]}}


def model(vocab, width, eps, layers):
    out = []
    for layer, mlp in layers:
        entry = copy.deepcopy(layer)
        entry["mlp"] = copy.deepcopy(mlp)
        out.append(entry)
    return {"architecture": "Suranex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": out}


YARN_A = {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 2.0}
YARN_B = {"factor": 1.5, "original": 48, "fast": 16.0, "slow": 0.5}

CONFIGS = {
    # odd sizes: nothing a multiple of 32; one expert a token; a layer without a feed-forward; heads
    # wider than their values and the other way round; no scaling, no squashing
    "odd": model(96, 48, 1e-5, [
        (rglru(40, 5, 3), moe(4, 1, 24, 1.0)),
        (attention(2, 1, 16, 8, 9, 3, 8, 100.0, 0.3), None),
        (attention(4, 4, 8, 16, 5, 0, 8, 50.0, 0.5, softcap=3.0), moe(3, 3, 8, 0.75, shared=(40, 3.0))),
    ]),
    # recurrent layers first and last, one block, two taps; a window larger than any prompt; no mask at all
    "mix": model(128, 64, 1e-6, [
        (rglru(64, 1, 2), moe(6, 3, 32, 2.5, shared=(64, 1.25))),
        (attention(4, 2, 32, 32, 20, 5, 16, 1000.0, 0.2, softcap=30.0, scaling=YARN_A), moe(6, 2, 32, 2.0)),
        (attention(2, 2, 32, 64, None, 0, 32, 1000.0, 0.1, softcap=10.0, scaling=YARN_B), None),
        (attention(8, 2, 16, 16, 300, 2, 4, 777.0, 0.25), moe(2, 1, 16, 1.0, shared=(16, 1.0))),
        (rglru(96, 3, 5), None),
    ]),
    # the sizes the matrix-core kernels take: heads of 64 with tiled bfloat16 pages of 64 tokens, widths of 32s
    "wide": model(200, 128, 1e-6, [
        (attention(4, 1, 64, 64, 70, 4, 64, 5000.0, 0.11, softcap=40.0, scaling=YARN_A), moe(4, 2, 64, 1.25, shared=(32, 2.5))),
        (rglru(128, 2, 3), moe(4, 2, 96, 1.25)),
        (attention(2, 2, 128, 128, 33, 17, 32, 5000.0, 0.09, softcap=20.0), moe(8, 4, 32, 3.0, shared=(64, 1.0))),
    ]),
}
PAGE = {"odd": 16, "mix": 32, "wide": 64}
LENGTHS = {"odd": [1, 23, 50, 9, 37, 64], "mix": [70, 3, 41, 129, 18], "wide": [150, 40, 97, 2, 66]}


def random_weights(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """Float32 weights by tensor name; values that bfloat16 holds exactly, so that both engines
    and the plain implementation read the same numbers."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, spec in tensor_specs_for(cfg).items():
        if spec.kind == "int":
            experts = int(cfg["layers"][int(name.split(".")[0][1:])]["mlp"]["router"]["experts"])  # "l<i>.mlp.table"
            out[name] = torch.rand((*spec.shape[:-1], experts), generator=g).argsort(-1)[..., : spec.shape[-1]].to(torch.int32)
            continue
        last = name.rsplit(".", 1)[-1]
        if "norm" in name:
            std = 0.3
        elif name.endswith(".lam"):
            std = 1.5
        elif name.endswith((".conv", ".ra", ".ri")):
            std = 0.4
        elif last == "b":
            std = 0.2
        elif name in ("embed",):
            std = 1.0
        else:
            std = 1.5 / (spec.shape[-1] ** 0.5)
        t = torch.randn(spec.shape, generator=g) * std
        if name.endswith((".q.norm", ".k.norm")):
            t = t + 1.0
        out[name] = t.to(torch.bfloat16).float()
    return out


def make_requests(cfg: dict, lengths: Sequence[int], seed: int) -> Dict[str, List[int]]:
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, cfg["vocab"], (n,), generator=g).tolist() for i, n in enumerate(lengths)}


def make_runner(cfg, weights, dtype, device, ops, page_size, num_pages, max_seqs=4, max_len=512) -> ModelRunner:
    eng = EngineConfig(page_size=page_size, num_pages=num_pages, max_num_seqs=max_seqs, max_model_len=max_len,
                       max_num_batched_tokens=max_len, dtype=dtype, device=device)
    m = build_model(cfg, eng, ops=ops)
    wd = torch.float32 if dtype == "float32" else torch.bfloat16
    m.load({k: (v if v.dtype == torch.int32 else v.to(wd)).to(device) for k, v in weights.items()})
    return ModelRunner(m, eng)


def plain_logits(cfg, weights, reqs) -> Dict[str, torch.Tensor]:
    return {rid: S.forward(cfg, weights, torch.tensor(toks)) for rid, toks in reqs.items()}


def relative_error(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Per position: the largest difference of the logits against the largest logit."""
    return (got.double() - want).abs().max(dim=1).values / want.abs().max(dim=1).values


F32_TOL = 3e-5
BF16_TOL = 6e-2


def assert_matches(got, want, bf16: bool, what: str) -> None:
    tol = BF16_TOL if bf16 else F32_TOL
    for rid, w in want.items():
        g = got[rid]
        assert g.shape == w.shape, f"{what}: request {rid} has {tuple(g.shape)} logits, expected {tuple(w.shape)}"
        assert torch.isfinite(g).all(), f"{what}: request {rid} has non-finite logits"
        err = relative_error(g, w)
        if (err > tol).any():
            first = int(torch.nonzero(err > tol)[0])
            raise AssertionError(f"{what}: request {rid} first differs at position {first} of {len(err)} "
                                 f"(relative error {err[first].item():.3e}, tolerance {tol:.1e}, largest {err.max().item():.3e})")
