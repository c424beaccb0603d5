"""Helpers of the Vurizen tests: small configurations, checkpoints on disk,
engines, and a driver that cuts sequences into steps."""

import json
import os
from typing import Dict, List, Optional, Sequence, Tuple

import torch
from safetensors.torch import save_file

import vurizen_oracle as oracle
from parallax_amd.models.config import ModelConfig
from parallax_amd.parallel.comm import CommContext
from parallax_amd.server.engine import Engine, EngineArgs


def moe_spec(experts=6, top=2, ff=24, groups=(3, 2), scale=1.5):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top, "scale": scale,
                       "groups": {"count": groups[0], "keep": groups[1]}}}


def gla_spec(heads=3, dim=24, vdim=40, tau=8.0, mlp="default"):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau},
            "mlp": moe_spec() if mlp == "default" else mlp}


def latent_spec(heads=3, dim=24, rot_dim=16, vdim=20, rank=40, window=9, scale=0.2,
                kv_from=None, rot_dims=None, base=500.0, scaling="default",
                mlp="default"):
    if scaling == "default":
        scaling = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim,
             "kv_rank": rank, "mask": {"size": window}, "scale": scale,
             "rot": {"dims": rot_dims or rot_dim, "base": base, "scaling": scaling}}
    if scaling is None:
        del mixer["rot"]["scaling"]
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": mixer,
            "mlp": moe_spec() if mlp == "default" else mlp}


def small_config(layers=None, width=48, vocab=97, mult=0.6, eps=1e-5) -> dict:
    """Sizes chosen away from powers of two: 3 heads, key dim 24, value dims
    40/20, rank 40, a rotated part of which only half the dims rotate, 6
    experts in 3 groups, a layer without feed-forward, a latent layer that
    reads an earlier layer's cache, and a latent layer first."""
    if layers is None:
        layers = [
            latent_spec(),
            gla_spec(),
            latent_spec(kv_from=0, heads=2, dim=16, vdim=24, window=5, mlp=None),
            gla_spec(heads=2, dim=40, vdim=24, tau=3.0, mlp=moe_spec(4, 1, 16, (1, 1), 1.0)),
            latent_spec(rot_dim=24, rot_dims=8, rank=24, window=33, scaling=None),
        ]
    return {"architecture": "Vurizen", "layers": layers, "norm": {"eps": eps},
            "residual_mult": mult, "vocab": vocab, "width": width}


def write_checkpoint(path: str, cfg: dict, weights: Dict[str, torch.Tensor]) -> str:
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in weights.items()},
              os.path.join(path, "model.safetensors"))
    return path


def make_engine(path: str, device="cpu", dtype=torch.float32, pages=64, block_size=8,
                max_requests=4, graphs=False, **kw) -> Engine:
    cfg = ModelConfig.from_pretrained(path)
    dev = torch.device(device)
    args = EngineArgs(block_size=block_size, num_kv_blocks=pages,
                      max_batch_size=max_requests, extra_linear_slots=0, dtype=dtype,
                      enable_prefix_cache=False, enable_graphs=graphs,
                      max_model_len=pages * block_size, **kw)
    comm = CommContext(world_size=1, rank=0, pp_size=1, tp_size=1, pp_rank=0,
                       tp_rank=0, device=dev)
    return Engine(cfg, args, comm=comm, model_path=path)


def run_schedule(engine: Engine, seqs: Dict[str, List[int]],
                 schedule: Sequence[Sequence[Tuple[str, int]]]) -> Dict[str, torch.Tensor]:
    """Feed the sequences step by step ([(name, count), ...] per step), asking
    for the logits of every position. Returns name -> [len, vocab] logits."""
    at = {k: 0 for k in seqs}
    got: Dict[str, List[torch.Tensor]] = {k: [] for k in seqs}
    for step in schedule:
        entries, end = [], []
        for name, count in step:
            lo = at[name]
            toks = seqs[name][lo : lo + count]
            entries.append((name, toks, list(range(len(toks)))))
            at[name] = lo + len(toks)
            if at[name] >= len(seqs[name]):
                end.append(name)
        out = engine.replay_step(entries, end).cpu()
        row = 0
        for name, toks, _ in entries:
            got[name].append(out[row : row + len(toks)])
            row += len(toks)
    return {k: torch.cat(v) for k, v in got.items() if v}


def oracle_logits(cfg: dict, weights, tokens: List[int]) -> torch.Tensor:
    return oracle.forward(cfg, weights, tokens).float()


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """Largest row error: rms of the difference (mean removed) over the rms of
    the wanted logits."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    scale = want.double().std().item()
    return float(d.pow(2).mean(-1).sqrt().max() / scale)


def row_errs(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / want.double().std()


def describe(got: torch.Tensor, want: torch.Tensor, tol: float) -> str:
    e = row_errs(got, want)
    bad = (e >= tol).nonzero().flatten().tolist()
    return "rows over %g: %s; values %s; median %.4f" % (
        tol, bad, [round(float(e[i]), 3) for i in bad], float(e.median()))


def close_in_bf16(got: torch.Tensor, want: torch.Tensor, tol: float) -> bool:
    """bf16 against the float64 reference: a sharp softmax or a router
    near-tie makes single positions far more sensitive to rounding than the
    rest, so: nine rows in ten within tol and the median row well inside it.
    (The float32 runs of the same kernels are held to rounding on every row,
    and same_as_whole() below is the sharper bf16 check.)"""
    e = row_errs(got, want)
    return bool((e < tol).double().mean() >= 0.9 and e.median() < tol / 3)


def same_as_whole(got: torch.Tensor, whole: torch.Tensor, tol: float = 0.02) -> bool:
    """A schedule's logits against the SAME engine dtype's logits for the
    sequence run alone and whole: the arithmetic is the same up to GEMM tile
    choices, so rows agree far inside bf16 rounding of the reference; 95 in
    100 must (a router near-tie may still flip here and there)."""
    e = row_errs(got, whole)
    return bool((e < tol).double().mean() >= 0.95)


def tokens(n: int, vocab: int, seed: int) -> List[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
