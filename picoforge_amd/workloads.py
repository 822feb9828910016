"""Seeded synthetic workloads at the measured shapes.

Shapes: hidden 2048, 512 routed experts, top-10, expert intermediate 512, one
shared expert of intermediate 512 with a sigmoid gate.  Everything here prepares
inputs; nothing computes the MoE block.
"""
import numpy as np

from . import abi
from .binding import Synth
from .layer import LayerWeights, rms_normalise

HIDDEN, EXPERTS, TOP_K, INTER, SHARED_INTER = 2048, 512, 10, 512, 512


def measured_config():
    return abi.moe_config(HIDDEN, EXPERTS, TOP_K, INTER, SHARED_INTER)


def layer_bytes(expert_type, cfg=None):
    """Stored bytes of one routed expert's gate + up rows and down rows, of the shared expert's, and of
    the two routers.  expert_type: a GGUF type for every expert tensor, or a checkpoint profile
    ("q2": IQ2_XXS gate/up, Q2_K down, Q8_0 shared; "q4": Q4_K gate/up, MXFP4 down, Q8_0 shared)."""
    cfg = cfg or measured_config()
    gate, down, shared = LayerWeights.PROFILE.get(expert_type, (expert_type,) * 3)

    def size(gtype, k, n):
        block, nbytes = abi.BLOCK[gtype]
        return k // block * nbytes * n
    h, i, s = cfg.hidden_size, cfg.intermediate, cfg.shared_intermediate
    return {"gate_up": 2 * size(gate, h, i), "down": size(down, cfg.down_physical, h),
            "shared_gate_up": 2 * size(shared, h, s), "shared_down": size(shared, s, h),
            "routers": (cfg.experts + 1) * h * 4}


def algorithmic_bytes_per_token(expert_type, unique_experts=TOP_K, cfg=None):
    """Bytes one decoded token must read: the selected experts' three tensors, the shared
    expert's, both routers (F32).  Q4_K: 23 666 688, IQ2_XXS: 13 123 584 at the measured shape."""
    b = layer_bytes(expert_type, cfg)
    return unique_experts * (b["gate_up"] + b["down"]) + b["shared_gate_up"] + b["shared_down"] + b["routers"]


def router_logits64(weights, x):
    cfg = weights.cfg
    router = weights.raw[0].view(np.float32).reshape(cfg.experts, cfg.hidden_size).astype(np.float64)
    return x.astype(np.float64) @ router.T


def top_margins(logits, k):
    top = -np.sort(-logits, axis=1)[:, :k + 1]
    return (top[:, :-1] - top[:, 1:]).min(axis=1)


def decode_tokens(weights, count, seed, min_margin=1e-3, max_margin=None):
    """`count` RMS-normalised N(0,1) activations whose sorted top-(k+1) router logits are at
    least min_margin apart (drawn, then kept or rejected), so expert selection does not depend
    on the order a logit is summed in.  max_margin keeps only tokens with a closer pair than that
    (tokens the kernels route again in the reference's order)."""
    synth, cfg = Synth(), weights.cfg
    kept, draw, drawn = [], 0, 0
    while sum(len(k) for k in kept) < count:
        x = rms_normalise(synth.normal((max(1024, count // 4), cfg.hidden_size), seed * 1000 + draw))
        draw += 1
        drawn += len(x)
        margins = top_margins(router_logits64(weights, x), cfg.top_k)
        ok = margins >= min_margin
        if max_margin is not None:
            ok &= margins < max_margin
        kept.append(x[ok])
    x = np.concatenate(kept)[:count]
    return np.ascontiguousarray(x), {"drawn": drawn, "kept_fraction": float(sum(len(k) for k in kept) / drawn)}


def verify_batches(weights, batches, seed, rho=0.85, min_margin=1e-3, group=4):
    """Groups of `group` consecutive tokens x_t = rho x_(t-1) + sqrt(1-rho^2) n_t (RMS-normalised), which
    makes adjacent tokens share about half of their top-10 experts; returns x [batches,group,H]
    and the achieved mean overlap and mean unique experts per batch."""
    synth, cfg = Synth(), weights.cfg
    out, overlaps, uniques, draw = [], [], [], 0
    while len(out) < batches:
        n = synth.normal((group * max(64, batches), cfg.hidden_size), seed * 1000 + draw).reshape(-1, group, cfg.hidden_size)
        draw += 1
        x = np.empty_like(n)
        x[:, 0] = n[:, 0]
        for t in range(1, group):
            x[:, t] = rho * x[:, t - 1] + np.sqrt(1 - rho * rho) * n[:, t]
        x = rms_normalise(x)
        z = router_logits64(weights, x.reshape(-1, cfg.hidden_size))
        ok = (top_margins(z, cfg.top_k) >= min_margin).reshape(-1, group).all(axis=1)
        ids = np.argsort(-z, axis=1, kind="stable")[:, :cfg.top_k].reshape(-1, group, cfg.top_k)
        for b in np.nonzero(ok)[0]:
            if len(out) == batches:
                break
            out.append(x[b])
            overlaps.append(np.mean([len(set(ids[b, t]) & set(ids[b, t + 1])) / cfg.top_k for t in range(group - 1)]))
            uniques.append(len(set(ids[b].reshape(-1))))
    return np.ascontiguousarray(np.stack(out)), {"mean_adjacent_overlap": float(np.mean(overlaps)),
                                                  "mean_unique_experts": float(np.mean(uniques))}


def zipf_router(weights, seed, s=1.1, temperature=1.0):
    """Rewrites column 0 of the router so that, with activation coordinate 0 held at 1.0, expert e
    gets a logit bias of -s * temperature * ln(rank_e): popularity follows a Zipf(s) profile.
    Returns the rank permutation used."""
    cfg = weights.cfg
    rng = np.random.default_rng(seed)
    rank = rng.permutation(cfg.experts) + 1
    router = weights.raw[0].view(np.float32).reshape(cfg.experts, cfg.hidden_size)
    router[:, 0] = (-s * temperature * np.log(rank)).astype(np.float32)
    return rank


def prefill_chunk(weights, tokens, seed, min_margin=0.0):
    """N(0,1) activations (not normalised) with coordinate 0 fixed at 1.0 (the bias input of zipf_router)."""
    x = Synth().normal((tokens, weights.cfg.hidden_size), seed * 1000 + 7)
    x[:, 0] = 1.0
    return x


def expert_load(weights, x):
    cfg = weights.cfg
    ids = np.argsort(-router_logits64(weights, x), axis=1, kind="stable")[:, :cfg.top_k]
    return np.bincount(ids.reshape(-1), minlength=cfg.experts)
