"""Helpers of the Zabusun tests: small irregular configurations. Checkpoint
writing, engines and the step driver are the ones of vurizen_util."""

from vurizen_util import (  # noqa: F401
    close_in_bf16, describe, make_engine, rel_err, row_errs, run_schedule,
    same_as_whole, tokens, write_checkpoint,
)


def dense(ff=56, limit=1.2):
    return {"kind": "dense", "ff": ff, "limit": limit}


def experts(n=5, top=2, ff=24, limit=2.0):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit},
            "router": {"experts": n, "top": top}}


def rot(dims, base=500.0, scaling="default"):
    if scaling == "default":
        scaling = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
    out = {"dims": dims, "base": base}
    if scaling is not None:
        out["scaling"] = scaling
    return out


def layer(heads=6, kv_heads=2, dim=12, vdim=20, scale=0.3, rotation="default",
          width=28, left_scale=0.7, right_scale=1.3, mlp="default"):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
            "scale": scale}
    if rotation == "default":
        rotation = rot(8)
    if rotation is not None:
        left["rot"] = rotation
    return {"type": "parallel",
            "mixer": {"left": left, "right": {"width": width},
                      "left_scale": left_scale, "right_scale": right_scale},
            "mlp": dense() if mlp == "default" else mlp}


def small_config(layers=None, width=40, vocab=83, eps=1e-5, logit_scale=0.7) -> dict:
    """Sizes away from powers of two and from each other: three query heads
    per kv head with key width 12 against value width 20 and 8 rotated
    dimensions; as many kv heads as heads with every dimension rotated and no
    frequency scaling; one kv head, no rotation and no feed-forward; dense
    and routed feed-forwards with one and two experts per token; recurrent
    widths 28, 52, 8 and 33."""
    if layers is None:
        layers = [
            layer(),
            layer(4, 4, 16, 8, 0.25, rot(16, 10000.0, None), 52, 1.0, 0.5, experts()),
            layer(3, 1, 24, 24, 0.2, None, 8, 0.4, 1.0, None),
            layer(2, 1, 8, 12, 0.35, rot(4, 100.0, {"factor": 2.0, "original": 16,
                                                     "fast": 4.0, "slow": 1.0}),
                  33, 1.5, 0.8, experts(3, 1, 16, 1.0)),
        ]
    return {"architecture": "Zabusun", "layers": layers, "norm": {"eps": eps},
            "vocab": vocab, "width": width, "logit_scale": logit_scale}
