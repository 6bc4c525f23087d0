"""Helpers of the Pudizen tests: small irregular configurations. Checkpoint
writing, engines and the step driver are the ones of vurizen_util."""

from vurizen_util import (  # noqa: F401
    close_in_bf16, describe, make_engine, rel_err, row_errs, run_schedule,
    same_as_whole, tokens, write_checkpoint,
)


def dense(ff=56):
    return {"kind": "dense", "ff": ff}


def rot(dims, base=500.0, scaling="default"):
    if scaling == "default":
        scaling = {"factor": 3.0, "low": 0.5, "high": 3.0, "original": 64}
    out = {"dims": dims, "base": base}
    if scaling is not None:
        out["scaling"] = scaling
    return out


def softmax_layer(heads=6, kv_heads=2, dim=12, vdim=20, scale=0.3, rotation="default",
                  mlp="default", window=None):
    """Type 'attention': whole-projection q/k norm, rotated values."""
    mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
          "rot": rot(8) if rotation == "default" else rotation}
    if window:
        mx["mask"] = {"size": window}
    return {"type": "attention", "mixer": mx, "mlp": dense() if mlp == "default" else mlp}


def window_layer(heads=4, kv_heads=1, dim=16, vdim=8, scale=0.25, window=9,
                 rotation="default", mlp="default"):
    """Type 'attention_2': sliding window, sigmoid key weights."""
    mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
          "mask": {"size": window}}
    if rotation == "default":
        rotation = rot(6, 300.0, None)
    if rotation is not None:
        mx["rot"] = rotation
    return {"type": "attention_2", "mixer": mx, "mlp": dense() if mlp == "default" else mlp}


def latent_layer(heads=3, dim=12, vdim=20, rank=24, scale=0.3, mlp="default"):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank,
                      "scale": scale},
            "mlp": dense() if mlp == "default" else mlp}


def small_config(layers=None, width=40, vocab=83, eps=1e-5, groups=5, scale=2.5,
                 buckets=61, mul_prev=13, mul_cur=5) -> dict:
    """Sizes away from powers of two and from each other: three query heads
    per kv head with key width 12 against value width 20 and 8 of 12
    dimensions rotated with scaled frequencies; a window of 9 over one kv
    head with 6 of 16 dimensions rotated; a latent of 24 under three heads; a
    window of 33 (several pages) with as many kv heads as heads and no
    feed-forward; all dimensions rotated and no scaling; five norm groups."""
    if layers is None:
        layers = [
            window_layer(),
            latent_layer(),
            softmax_layer(),
            window_layer(3, 3, 8, 12, 0.35, 33, rot(8, 100.0, {"factor": 2.0, "low": 1.0,
                                                              "high": 2.0, "original": 16}),
                         None),
            softmax_layer(4, 4, 16, 8, 0.25, rot(16, 10000.0, None), dense(24)),
            latent_layer(2, 8, 8, 40, 0.2, None),
        ]
    return {"architecture": "Pudizen", "layers": layers,
            "norm": {"eps": eps, "groups": groups},
            "embedding": {"scale": scale,
                          "bigram": {"buckets": buckets, "mul_prev": mul_prev,
                                     "mul_cur": mul_cur}},
            "vocab": vocab, "width": width}
