"""Shared pieces of the Bokulorn tests: small configurations made here (none of them a real model's
sizes), the engine or single kernels on one side, oracle/bokulorn_oracle.py on the other. Replay, step
and comparison helpers are the ones of tests/_kagalorn.py."""
from __future__ import annotations

from tests._kagalorn import TOL, assert_close, make_step, rel_err, replay, tokens_for, write_model  # noqa: F401

MOE_A = {"kind": "moe", "expert": {"ff": 20}, "router": {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 2}}}
MOE_B = {"kind": "moe", "expert": {"ff": 12}, "router": {"experts": 4, "top": 2}}
LAT_A = {"heads": 3, "dim": 12, "rot_dim": 8, "rot": {"base": 5000.0, "dims": 8}, "vdim": 10, "q_rank": 20, "kv_rank": 24,
         "scale": 0.2}
LAT_B = {"heads": 2, "dim": 16, "vdim": 8, "q_rank": 12, "kv_rank": 20, "scale": 0.25}
DEL_A = {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 12, "conv": 3, "decay_rank": 5, "gate_rank": 6}

CFG_MAIN = {
    "architecture": "Bokulorn", "vocab": 67, "width": 48, "norm": {"eps": 1e-5}, "embedding": {"scale": 3.5},
    "layers": [
        {"type": "latent_attention", "mixer": LAT_A, "mlp": MOE_A},
        {"type": "channel_delta", "mixer": DEL_A, "mlp": MOE_B},
        {"type": "latent_attention_2", "mixer": LAT_B, "mlp": None},
        {"type": "latent_attention", "mixer": LAT_A, "mlp": MOE_A, "weights_of": 0},
        {"type": "channel_delta", "mixer": DEL_A, "mlp": MOE_B, "weights_of": 1},
    ],
}
# values that a model may happen to make 1 or equal: one head, one kv head under two heads, one tap, thin factors of
# rank one, a latent wider than a wave, every expert chosen, one expert chosen, groups of one expert, no groups,
# a positional layer without a rotated part, a rotation over part of the positional entries, a layer that borrows
# the weights of a later one, no embedding scale
ODD_LAT = {"heads": 1, "dim": 4, "rot_dim": 6, "rot": {"base": 100.0, "dims": 2}, "vdim": 5, "q_rank": 7, "kv_rank": 70,
           "scale": 0.5}
ODD_DEL = {"heads": 2, "kv_heads": 1, "dim": 40, "vdim": 70, "conv": 1, "decay_rank": 1, "gate_rank": 1}
ODD_LAT2 = {"heads": 5, "dim": 3, "vdim": 3, "q_rank": 5, "kv_rank": 9, "scale": 0.6}
CFG_ODD = {
    "architecture": "Bokulorn", "vocab": 37, "width": 40, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "latent_attention_2", "mixer": ODD_LAT2, "mlp": None, "weights_of": 3},
        {"type": "latent_attention", "mixer": ODD_LAT,
         "mlp": {"kind": "moe", "expert": {"ff": 8}, "router": {"experts": 3, "top": 3, "groups": {"count": 1, "keep": 1}}}},
        {"type": "channel_delta", "mixer": ODD_DEL,
         "mlp": {"kind": "moe", "expert": {"ff": 16}, "router": {"experts": 5, "top": 1, "groups": {"count": 5, "keep": 2}}}},
        {"type": "latent_attention_2", "mixer": ODD_LAT2, "mlp": None},
        {"type": "latent_attention", "mixer": {"heads": 2, "dim": 8, "vdim": 8, "q_rank": 8, "kv_rank": 8, "scale": 0.35},
         "mlp": {"kind": "moe", "expert": {"ff": 8}, "router": {"experts": 2, "top": 1}}},
    ],
}
# latent and positional sizes in multiples of 16 (in bf16 the attention then runs on the matrix cores; 48 = one
# 32-wide and one 16-wide step over the key row), five query heads on the one cached row
CFG_WIDE = {
    "architecture": "Bokulorn", "vocab": 83, "width": 64, "norm": {"eps": 1e-6}, "embedding": {"scale": 8.0},
    "layers": [
        {"type": "latent_attention", "mixer": {"heads": 5, "dim": 32, "rot_dim": 16, "rot": {"base": 10000.0, "dims": 16},
                                               "vdim": 32, "q_rank": 48, "kv_rank": 32, "scale": 0.14},
         "mlp": {"kind": "moe", "expert": {"ff": 32}, "router": {"experts": 8, "top": 3, "groups": {"count": 4, "keep": 2}}}},
        {"type": "channel_delta", "mixer": {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 32, "conv": 4, "decay_rank": 8,
                                            "gate_rank": 4}, "mlp": None},
        {"type": "latent_attention_2", "mixer": {"heads": 4, "dim": 16, "vdim": 16, "q_rank": 32, "kv_rank": 64, "scale": 0.25},
         "mlp": {"kind": "moe", "expert": {"ff": 32}, "router": {"experts": 8, "top": 3, "groups": {"count": 4, "keep": 2}}}},
    ],
}


def random_config(seed: int) -> dict:
    """A configuration drawn from lists of sizes (latent and positional sizes in and out of the multiples of 16 that
    the matrix-core kernel takes, one to eight heads, two to four taps, four to sixteen experts), six layers in
    random order, two of which borrow another layer's weights."""
    import random
    r = random.Random(seed)
    width = r.choice([64, 96, 160])

    def moe():
        if r.random() < 0.2:
            return None
        count = r.choice([1, 2, 4])
        experts = count * r.choice([1, 2, 4]) if count > 1 else r.choice([4, 6, 8])
        top = r.randint(1, max(1, min(4, experts // 2)))
        keep = r.randint(max(1, -(-top // (experts // count))), count)
        router = {"experts": experts, "top": top}
        if count > 1 or r.random() < 0.5:
            router["groups"] = {"count": count, "keep": keep}
        return {"kind": "moe", "expert": {"ff": r.choice([24, 32, 64])}, "router": router}

    def mixer(kind):
        if kind == "channel_delta":
            kv = r.choice([1, 2, 3])
            return {"heads": kv * r.choice([1, 2]), "kv_heads": kv, "dim": r.choice([16, 24, 32, 64]), "vdim": r.choice([16, 40, 64]),
                    "conv": r.choice([2, 3, 4]), "decay_rank": r.choice([4, 9]), "gate_rank": r.choice([3, 8])}
        m = {"heads": r.randint(1, 8), "dim": r.choice([8, 24, 32, 64]), "vdim": r.choice([8, 24, 32]),
             "q_rank": r.choice([16, 40, 64]), "kv_rank": r.choice([16, 48, 80, 100]), "scale": r.choice([0.1, 0.2, 0.3])}
        if kind == "latent_attention":
            m["rot_dim"] = r.choice([8, 16, 32])
            m["rot"] = {"base": r.choice([1000.0, 10000.0, 50000.0]), "dims": m["rot_dim"]}
        return m

    layers = []
    for i in range(4):
        kind = r.choice(["latent_attention", "latent_attention_2", "channel_delta"])
        layers.append({"type": kind, "mixer": mixer(kind), "mlp": moe()})
    for _ in range(2):
        j = r.randrange(4)
        layers.insert(r.randint(j + 1, len(layers)), {**layers[j], "weights_of": j})
    # indices moved with the insertions: name the sources again
    own = [i for i, L in enumerate(layers) if "weights_of" not in L]
    for i, L in enumerate(layers):
        if "weights_of" in L:
            L["weights_of"] = next(k for k in own if layers[k]["mixer"] is L["mixer"])
    return {"architecture": "Bokulorn", "vocab": r.choice([50, 131]), "width": width, "norm": {"eps": r.choice([1e-6, 1e-5])},
            "embedding": {"scale": r.choice([1.0, width ** 0.5])}, "layers": layers}
