"""A synthetic MoE decoder step built from the C-ABI operators: per layer

    h   = q8k(rmsnorm(x))                              mq_rmsnorm_mul_mat_q4k (with the previous residual add; one launch
    qkv = W_qkv . h                                                            at one token; wq, wk, wv stacked row-wise)
    o   = W_o . q8k(qkv[:, :n_q])                      mq_mul_mat_q4k     (the attention core itself is not on
                                                                           this path: q stands in for its output)
    x   = x + o ; h2 = rmsnorm(x)                      mq_add_rmsnorm_router_f32 (one launch; mq_add_rmsnorm_f32 +
    logits = W_router . h2                                                        mq_router_logits_f32 for hidden > 4096)
    y   = moe_layer(h2, logits) (+ shared expert)      mq_moe_layer_q4k
    x   = x + y                                        (fused into the next layer's first call)

which is the operator sequence of a Qwen3.5-35B-A3B-class layer in the reference's graph
(core/src/llm/graph/decoder.cpp:2265, :2426-2600; core/src/llm/moe/native.cpp:4831-4911) with the
attention core left out.  Weights are random-init Q4_K generated on the device from seeds.  The
whole step can be captured in one HIP graph (torch.cuda.CUDAGraph) and replayed.

FusedDecodeStep runs the same layers through mq_decoder_step: one persistent kernel for the whole run of
layers (n <= 8), whose results are bit-identical to DecodeStep's.
"""
import ctypes as C
from dataclasses import dataclass

import torch

from . import _lib, ops, synth


@dataclass
class StepConfig:
    n_layers: int = 40
    hidden: int = 2048
    n_experts: int = 256
    inter: int = 512
    top_k: int = 8
    n_q: int = 2048        # 16 query heads x 128
    n_kv: int = 256        # 2 KV heads x 128
    shared_expert: bool = True
    eps: float = 1e-6
    seed: int = 2026
    # True: every layer routes on resident N(0,1) logits (the MoE block as the benchmark config states it),
    # the router projection still runs but its output is not used.  False: logits = W_router . rmsnorm(x).
    synthetic_logits: bool = False

    def layer_weight_bytes(self) -> int:
        """ggml bytes of one layer's weights (Q4_K: 144 B per 256 weights; router fp32)."""
        q4 = lambda r, c: r * c // 256 * 144
        b = self.n_experts * (2 * q4(self.inter, self.hidden) + q4(self.hidden, self.inter))
        if self.shared_expert:
            b += 2 * q4(self.inter, self.hidden) + q4(self.hidden, self.inter)
        b += q4(self.n_q + 2 * self.n_kv, self.hidden) + q4(self.hidden, self.n_q)
        return b + self.n_experts * self.hidden * 4


class Layer:
    def __init__(self, cfg: StepConfig, index: int):
        s = lambda name: synth.tensor_seed("decode-step", cfg.seed, index, name)
        H, I, E = cfg.hidden, cfg.inter, cfg.n_experts
        self.wqkv = ops.Q4KWeight.synthetic(s("wqkv"), cfg.n_q + 2 * cfg.n_kv, H)
        self.wo = ops.Q4KWeight.synthetic(s("wo"), H, cfg.n_q)
        self.gate_exps = ops.Q4KWeight.synthetic(s("gate_exps"), I, H, E)
        self.up_exps = ops.Q4KWeight.synthetic(s("up_exps"), I, H, E)
        self.down_exps = ops.Q4KWeight.synthetic(s("down_exps"), H, I, E)
        self.shared = None
        if cfg.shared_expert:
            self.shared = (ops.Q4KWeight.synthetic(s("sh_gate"), I, H), ops.Q4KWeight.synthetic(s("sh_up"), I, H),
                           ops.Q4KWeight.synthetic(s("sh_down"), H, I))
        g = torch.Generator(device="cuda").manual_seed(s("router") & 0x7FFFFFFF)
        self.router = torch.randn((E, H), device="cuda", generator=g) * (1.0 / H ** 0.5)
        self.sh_gate_inp = torch.randn((H,), device="cuda", generator=g) * (1.0 / H ** 0.5) if cfg.shared_expert else None
        self.desc = _lib.MoELayerDesc(
            self.gate_exps._h, self.up_exps._h, self.down_exps._h,
            self.shared[0]._h if self.shared else None, self.shared[1]._h if self.shared else None,
            self.shared[2]._h if self.shared else None,
            self.sh_gate_inp.data_ptr() if self.sh_gate_inp is not None else None,
            cfg.top_k, ops.SILU_EXACT, ops.ROUTE_FLOOR)

    def free(self):
        for w in (self.wqkv, self.wo, self.gate_exps, self.up_exps, self.down_exps) + (self.shared or ()):
            w.free()


class DecodeStep:
    """Owns the weights of `cfg.n_layers` layers and the activation buffers of one batch width."""

    def __init__(self, cfg: StepConfig, n_tokens: int, layers=None):
        self.cfg, self.n = cfg, n_tokens
        self._owns_layers = layers is None
        self.layers = layers if layers is not None else [Layer(cfg, i) for i in range(cfg.n_layers)]
        f = lambda *shape: torch.empty(shape, dtype=torch.float32, device="cuda")
        H = cfg.hidden
        self.x, self.h, self.o, self.y = f(n_tokens, H), f(n_tokens, H), f(n_tokens, H), f(n_tokens, H)
        self.x_alt = f(n_tokens, H)
        self.qkv = f(n_tokens, cfg.n_q + 2 * cfg.n_kv)
        self.logits = f(n_tokens, cfg.n_experts)
        self.ids = torch.empty((cfg.n_layers, n_tokens, cfg.top_k), dtype=torch.int32, device="cuda")
        self.wts = f(cfg.n_layers, n_tokens, cfg.top_k)
        self.out = f(n_tokens, H)
        self.h_q8 = ops.Q8KActs(n_tokens, H)
        self.fixed_logits = None
        if cfg.synthetic_logits:
            g = torch.Generator(device="cuda").manual_seed(synth.tensor_seed("decode-step-logits", cfg.seed, n_tokens) & 0x7FFFFFFF)
            self.fixed_logits = torch.randn((cfg.n_layers, n_tokens, cfg.n_experts), device="cuda", generator=g)
        self._graph = None

    def silu_mode(self) -> int:
        # decode widths use the exact exponential, wider ones the polynomial (core/src/llm/moe/native.cpp:3614-3616)
        return ops.SILU_EXACT if self.n <= 4 else ops.SILU_FAST

    def run(self, x_in: torch.Tensor) -> torch.Tensor:
        """One step, eagerly launched on the current stream."""
        self.x.copy_(x_in)
        self._launch()
        return self.out

    def _launch(self) -> None:
        L, cfg, n = _lib.lib(), self.cfg, self.n
        st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        p = lambda t: C.c_void_p(t.data_ptr())
        chk = _lib.check
        delta = None
        x, x_next = self.x, self.x_alt   # the residual stream alternates between two buffers (see below)
        fused_router = cfg.hidden % 256 == 0 and cfg.hidden <= 4096
        for i, ly in enumerate(self.layers):
            ly.desc.silu_mode = self.silu_mode()
            # residual add, norm, Q8_K and the qkv projection (one launch at one token); the sum goes to the other buffer
            chk(L.mq_rmsnorm_mul_mat_q4k(ly.wqkv._h, p(x), p(delta) if delta is not None else None, None, n, C.c_float(cfg.eps),
                                         p(x_next), p(self.qkv), self.qkv.shape[1], st), "mq_rmsnorm_mul_mat_q4k")
            x, x_next = x_next, x
            chk(L.mq_mul_mat_q4k(ly.wo._h, p(self.qkv), n, self.qkv.shape[1], p(self.o), cfg.hidden, st), "wo")
            if fused_router:
                # residual add, norm and router projection in one launch; its sum goes to the other buffer because
                # every workgroup of a row reads x while one of them writes the sum
                chk(L.mq_add_rmsnorm_router_f32(p(x), p(self.o), None, n, cfg.hidden, C.c_float(cfg.eps), p(x_next), p(self.h),
                                                p(ly.router), cfg.n_experts, p(self.logits), st), "mq_add_rmsnorm_router_f32")
                x, x_next = x_next, x
            else:
                chk(L.mq_add_rmsnorm_f32(p(x), p(self.o), None, n, cfg.hidden, C.c_float(cfg.eps), p(x), p(self.h), st),
                    "mq_add_rmsnorm_f32")
                chk(L.mq_router_logits_f32(p(ly.router), cfg.n_experts, cfg.hidden, p(self.h), n, cfg.hidden,
                                           p(self.logits), st), "mq_router_logits_f32")
            lg = self.fixed_logits[i] if self.fixed_logits is not None else self.logits
            chk(L.mq_moe_layer_q4k(C.byref(ly.desc), p(self.h), p(lg), n, p(self.y), p(self.ids[i]),
                                   p(self.wts[i]), st), "mq_moe_layer_q4k")
            delta = self.y
        # final residual add; the normalised copy lands in self.h and is not used
        chk(L.mq_add_rmsnorm_f32(p(x), p(delta), None, n, cfg.hidden, C.c_float(cfg.eps), p(self.out), p(self.h),
                                 st), "mq_add_rmsnorm_f32")

    def capture(self) -> None:
        """Capture the step into a HIP graph (after one eager run has sized every workspace)."""
        self._launch()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            self._launch()
        self._graph = g

    def replay(self) -> torch.Tensor:
        self._graph.replay()
        return self.out

    def free(self):
        self._graph = None
        self.h_q8.free()
        if self._owns_layers:
            for ly in self.layers:
                ly.free()
        self.layers = []


class FusedDecodeStep:
    """The layers of a DecodeStep through mq_decoder_step (one launch per step, n <= 8 tokens)."""

    def __init__(self, cfg: StepConfig, n_tokens: int, layers, fixed_logits=None):
        self.cfg, self.n, self.layers = cfg, n_tokens, layers
        f = lambda *shape: torch.empty(shape, dtype=torch.float32, device="cuda")
        self.x, self.out = f(n_tokens, cfg.hidden), f(n_tokens, cfg.hidden)
        self.ids = torch.empty((len(layers), n_tokens, cfg.top_k), dtype=torch.int32, device="cuda")
        self.wts = f(len(layers), n_tokens, cfg.top_k)
        self.fixed_logits = fixed_logits          # [n_layers, n_tokens, n_experts] or None
        table = (_lib.DecoderLayerDesc * len(layers))()
        for i, ly in enumerate(layers):
            table[i].wqkv, table[i].wo = ly.wqkv._h, ly.wo._h
            table[i].attn_norm_dev = table[i].ffn_norm_dev = None
            table[i].router_dev = ly.router.data_ptr()
            table[i].fixed_logits_dev = fixed_logits[i].data_ptr() if fixed_logits is not None else None
            table[i].moe = ly.desc
        h = C.c_void_p()
        _lib.check(_lib.lib().mq_decoder_create(table, len(layers), n_tokens, C.c_float(cfg.eps), C.byref(h)),
                   "mq_decoder_create")
        self._h = h
        self._graph = None

    def _launch(self) -> None:
        p = lambda t: C.c_void_p(t.data_ptr())
        st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        _lib.check(_lib.lib().mq_decoder_step(self._h, p(self.x), self.n, -1, p(self.out), p(self.ids), p(self.wts), st),
                   "mq_decoder_step")

    def run(self, x_in: torch.Tensor) -> torch.Tensor:
        self.x.copy_(x_in)
        self._launch()
        return self.out

    def status(self) -> None:
        """Synchronise and raise if a step abandoned a device-wide barrier."""
        _lib.check(_lib.lib().mq_decoder_status(self._h), "mq_decoder_status")

    def capture(self) -> None:
        self._launch()
        self.status()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            self._launch()
        self._graph = g

    def replay(self) -> torch.Tensor:
        self._graph.replay()
        return self.out

    def free(self) -> None:
        self._graph = None
        if self._h:
            _lib.lib().mq_decoder_free(self._h)
            self._h = None
