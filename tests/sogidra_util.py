"""Helpers of the Sogidra tests: small irregular configurations. Checkpoint
writing, engines and the step driver are the ones of vurizen_util."""

from vurizen_util import (  # noqa: F401
    close_in_bf16, describe, make_engine, rel_err, row_errs, run_schedule,
    same_as_whole, tokens, write_checkpoint,
)


def dense(ff=56):
    return {"kind": "dense", "ff": ff}


def diff_spec(heads=4, kv_heads=2, dim=12, vdim=20, scale=0.3, diff=0.2,
              coef=0.4, every=7, kv_from=None, mlp="default"):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
             "scale": scale, "diff": diff, "q_temp": {"coef": coef, "every": every}}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "attention", "mixer": mixer,
            "mlp": dense() if mlp == "default" else mlp}


def window_spec(heads=6, kv_heads=2, dim=16, scale=0.4, softcap=8.0, size=11,
                pool=3, mlp="default"):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim,
             "scale": scale, "softcap": softcap,
             "mask": {"size": size, "pool": pool}}
    return {"type": "attention_2", "mixer": mixer,
            "mlp": dense() if mlp == "default" else mlp}


def small_config(layers=None, width=40, vocab=83, eps=1e-5, max_positions=256) -> dict:
    """Sizes away from powers of two and from each other: three heads per kv
    head in the windowed layers and two in the differential ones, key width
    12 against value width 20, pooled blocks of 3 and 5 tokens (neither
    divides a page of 8), a layer without feed-forward, a differential layer
    that reads an earlier one's rows, and a windowed layer first."""
    if layers is None:
        layers = [
            window_spec(),
            diff_spec(),
            window_spec(heads=2, kv_heads=2, dim=24, size=4, pool=5, softcap=3.0,
                        mlp=None),
            diff_spec(heads=6, kv_heads=2, kv_from=1, scale=0.5, coef=0.1,
                      every=3, mlp=dense(24)),
            window_spec(heads=3, kv_heads=1, dim=8, size=30, pool=8),
        ]
    return {"architecture": "Sogidra", "layers": layers, "norm": {"eps": eps},
            "vocab": vocab, "width": width, "max_positions": max_positions}
