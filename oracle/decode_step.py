"""CPU restatement of the synthetic decoder step (TEST INFRASTRUCTURE ONLY, like everything in oracle/).

Composes the C oracle's Q4_K x Q8_K operators with numpy versions of the two fp32 operators around
them, in the operator order of densecore_amd/decode_step.py:
  * add + RMSNorm: core/tests/kernels/test_normalization.cpp:57-68 (the reference's own plain
    restatement of AddRMSNorm, core/src/kernels/hwy/hwy_normalization.cc:102-153), unit weight;
  * router logits: an fp32 matrix-vector product accumulated in double (ggml's F32 mul_mat order is not
    reproduced; the fp32 results agree to rounding);
  * MoE layer, dense projections: q4k_oracle.c.
"""
import numpy as np

from . import binding as orc


def add_rmsnorm(x, delta, eps):
    s = x if delta is None else (x + delta).astype(np.float32)
    ssq = np.sum(s.astype(np.float64) ** 2, axis=1, keepdims=True)
    scale = (1.0 / np.sqrt((ssq / s.shape[1]).astype(np.float32) + np.float32(eps))).astype(np.float32)
    return s, (s * scale).astype(np.float32)


def router_logits(w_router, h):
    return (h.astype(np.float64) @ w_router.astype(np.float64).T).astype(np.float32)


def layer_forward(lw: dict, x, delta, cfg, silu, order=orc.ORDER_DOTPROD, fixed_logits=None):
    """One layer on host weights `lw` (ggml-layout uint8 arrays + fp32 router).  Returns the stage outputs.
    fixed_logits: route on these [n, n_experts] instead of on the router projection (which is still returned)."""
    H, I = cfg.hidden, cfg.inter
    x1, h = add_rmsnorm(x, delta, cfg.eps)
    qkv = orc.mul_mat_q4k_f32(lw["wqkv"], H, h, order)
    o = orc.mul_mat_q4k_f32(lw["wo"], cfg.n_q, np.ascontiguousarray(qkv[:, :cfg.n_q]), order)
    x2, h2 = add_rmsnorm(x1, o, cfg.eps)
    logits = router_logits(lw["router"], h2)
    shared = (lw["sh_gate"], lw["sh_up"], lw["sh_down"], lw["sh_gate_inp"]) if "sh_gate" in lw else None
    moe = orc.moe_layer(lw["gate_exps"], lw["up_exps"], lw["down_exps"], H, I, cfg.top_k, h2,
                        logits if fixed_logits is None else fixed_logits, shared, order, silu, 1, 0)
    return {"h": h, "qkv": qkv, "o": o, "x": x2, "h2": h2, "logits": logits, "y": moe["y"], "ids": moe["ids"],
            "weights": moe["weights"]}
