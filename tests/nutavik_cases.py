"""Small Nutavik configurations that differ from each other in every size and option, random
weights for them, and helpers to run them through the engine and the plain implementation."""
from __future__ import annotations

import copy
from typing import Dict, List, Sequence

import torch

import plain_nutavik as P
from yalis_amd.config.runtime import EngineConfig
from yalis_amd.engine.factory import build_model, tensor_specs_for
from yalis_amd.engine.step import ModelRunner


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, base, scale, scaling=None, kv_from=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale,
         "rot": {"base": base, "dims": rot_dim, "scaling": scaling}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m}


def delta(heads, kv_heads, dim, vdim, conv):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


def gla(heads, dim, vdim, tau, low_rank=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}
    if low_rank is not None:
        m["low_rank"] = low_rank
    return {"type": "gla", "mixer": m}


def model(vocab, width, eps, mult, logit_scale, layers):
    out = []
    for layer, ff in layers:
        entry = copy.deepcopy(layer)
        entry["mlp"] = None if ff is None else {"kind": "dense", "ff": ff}
        out.append(entry)
    return {"architecture": "Nutavik", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult,
            "logit_scale": logit_scale, "layers": out}


YARN_A = {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 2.0}
YARN_B = {"factor": 1.5, "original": 48, "fast": 16.0, "slow": 0.5}

CONFIGS = {
    # nothing a multiple of 8; a recurrent layer first; one head; a layer without feed-forward; a borrowed
    # cache read with other heads; multiplier and logit scale both 1
    "odd": model(70, 40, 1e-5, 1.0, 1.0, [
        (delta(4, 2, 12, 10, 3), 24),
        (latent(3, 10, 6, 14, 20, 12, 100.0, 0.3), None),
        (gla(1, 20, 6, 4.0, low_rank=5), 36),
        (latent(5, 4, 6, 8, 20, 9, 100.0, 0.45, kv_from=1), 12),
    ]),
    # two caches of different row lengths, each read by a later layer too; one tap; value heads sharing keys
    "mix": model(128, 64, 1e-6, 0.5, 3.0, [
        (gla(4, 16, 16, 7.5), 32),
        (latent(2, 32, 8, 16, 24, 40, 1000.0, 0.2, scaling=YARN_A), 48),
        (delta(2, 2, 32, 48, 2), None),
        (latent(6, 8, 16, 8, 48, 16, 500.0, 0.35, scaling=YARN_B), 32),
        (latent(4, 16, 8, 24, 24, 32, 1000.0, 0.25, scaling=YARN_A, kv_from=1), None),
        (delta(8, 2, 8, 8, 1), 64),
        (latent(1, 24, 16, 40, 48, 8, 500.0, 0.15, scaling=YARN_B, kv_from=3), 16),
    ]),
    # sizes of whole wavefronts: keys of 128 channels (eight lanes to a column of the state), latents of 128
    "wide": model(200, 128, 1e-6, 0.25, 0.5, [
        (latent(8, 64, 32, 64, 128, 96, 5000.0, 0.1, scaling=YARN_A), 256),
        (delta(4, 2, 64, 64, 4), 128),
        (gla(2, 128, 64, 16.0, low_rank=8), None),
        (latent(4, 32, 32, 128, 128, 64, 5000.0, 0.12, scaling=YARN_A, kv_from=0), 128),
    ]),
}
PAGE = {"odd": 16, "mix": 32, "wide": 64}
LENGTHS = {"odd": [1, 23, 50, 9, 37, 64], "mix": [70, 3, 41, 129, 18], "wide": [150, 40, 97, 2, 66]}


def random_weights(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """Float32 weights by tensor name; values that bfloat16 holds exactly, so that both engines and
    the plain implementation read the same numbers."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, spec in tensor_specs_for(cfg).items():
        last = name.rsplit(".", 1)[-1]
        is_norm_weight = last == "norm" or last.startswith("norm")
        if name.endswith(".b") and ("norm" in name.rsplit(".", 2)[-2] or name.endswith("a2.b")):
            std = 0.2 if "norm" in name else 1.0  # a norm's bias; the decay's bias
        elif is_norm_weight:
            std = 0.3
        elif last == "conv":
            std = 0.5
        elif last in ("A_log", "dt_bias"):
            std = 0.7
        elif name == "embed":
            std = 1.0
        else:
            std = 1.5 / (spec.shape[-1] ** 0.5)
        t = torch.randn(spec.shape, generator=g) * std
        if is_norm_weight:
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
    m.load({k: v.to(wd).to(device) for k, v in weights.items()})
    return ModelRunner(m, eng)


def plain_logits(cfg, weights, reqs) -> Dict[str, torch.Tensor]:
    return {rid: P.forward(cfg, weights, torch.tensor(toks)) for rid, toks in reqs.items()}


def relative_error(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Per position: the root mean square of the logits' difference (its mean taken off) against that of the logits."""
    d = got.double() - want
    d = d - d.mean(dim=1, keepdim=True)
    w = want - want.mean(dim=1, keepdim=True)
    return d.pow(2).mean(dim=1).sqrt() / w.pow(2).mean(dim=1).sqrt().clamp_min(1e-30)


F32_TOL = 1e-4
# bfloat16 against the unrounded float64 implementation: the design divides each head's read-out by its
# root mean square, so where a read-out is nearly nothing (a first token whose q . k almost cancels) the
# rounding of q and k decides its sign and that position's logits; such positions are few.  Most positions
# stay under BF16_TOL, none is beyond BF16_WORST (unrelated logits are 1.4 apart), and the float32 engine
# pins the arithmetic itself.
BF16_TOL = 6e-2
BF16_FEW = 0.1
BF16_WORST = 0.6


def assert_matches(got, want, bf16: bool, what: str) -> None:
    over = total = 0
    for rid, w in want.items():
        g = got[rid]
        assert g.shape == w.shape, f"{what}: request {rid} has {tuple(g.shape)} logits, expected {tuple(w.shape)}"
        assert torch.isfinite(g).all(), f"{what}: request {rid} has non-finite logits"
        err = relative_error(g, w)
        tol = BF16_WORST if bf16 else F32_TOL
        if (err > tol).any():
            first = int(torch.nonzero(err > tol)[0])
            raise AssertionError(f"{what}: request {rid} first differs at position {first} of {len(err)} "
                                 f"(relative error {err[first].item():.3e}, tolerance {tol:.1e}, largest {err.max().item():.3e})")
        over += int((err > BF16_TOL).sum())
        total += len(err)
    if bf16:
        assert over <= max(1, BF16_FEW * total), f"{what}: {over} of {total} positions differ by more than {BF16_TOL:.1e}"
