"""Verozen: a decoder-only model on an fp32 residual stream that norms AFTER every residual sum
(x <- N(c x + sublayer(x)), N a grouped RMS norm), whose layers mix tokens by one of three mechanisms -- gated linear
attention (a decay per key channel), causal attention with sigmoid weights whose values are the raw keys, retention (a
fixed decay per head) -- feed forward through a grouped top-k mixture of erf-GELU experts, and take a per-layer slice of
a second token embedding as a gated, normed low-rank input after the feed-forward.  (No counterpart in the reference;
the module layout follows its model files, python/sglang/srt/models/deepseek_v2.py for the mixture.)

Per layer (T tokens, width D), besides the GEMMs' own launches:

  in_proj(h)               every projection of the mixer's input in one GEMM         gla: q | k | v | g | a1   ret: q | k | v | g   att: q | k
  gla        a2(a1 h) -> fp32 gate logits; LinearRecurrence (decay from the logits inside); HeadNormGate; o
  retention  HeadNormRope on q and on k (fp32 out, k scaled); LinearRecurrence; HeadNormGate; o
  attention  HeadNormRope on q; on k straight into the key cache; raw k into the value cache; SigmoidAttention; o
  GroupRMSNorm             x <- N(c x + mixer) and its activation-dtype copy h                           1 launch, fp32
  router, experts          fp32 logits GEMM, route, align, two grouped GEMMs                              5 launches
  GroupRMSNorm             x <- N(c x + sum_j w_j expert_j) and h                                         1 launch, fp32
  token side               gate GEMM, gelu_tanh(.) * table[token, slice], proj GEMM, x += RMSnorm(y) w    4 launches

Norms, rotation angles, attention scores / weights, decays, recurrent state, router and the residual sum are fp32 in every
dtype; `dtype` is what the projections read and write.  Every size comes from the configuration, layer by layer.
Tensor parallelism is not implemented for this family (its head counts need not divide)."""
from typing import Dict

import torch
from torch import nn

from ..distributed.parallel_state import get_tensor_model_parallel_world_size
from ..layers.linear import ReplicatedLinear
from ..layers.linear_recurrence import HeadNormGate, HeadNormRope, LinearRecurrence
from ..layers.logits_processor import LogitsProcessor
from ..layers.moe import GroupedExperts, GroupedTopKRouter
from ..layers.post_norm import GroupRMSNorm, NormedResidualAdd
from ..layers.sigmoid_attention import SigmoidAttention
from ..layers.vocab_parallel_embedding import ParallelLMHead
from ..ops_backend import get_ops


DEFAULT_GATE_RANK = 16     # rank of the decay projection of a gated-linear-attention layer built without a checkpoint


def _rot(mx: dict):
    rot = mx.get("rot") or {}
    return int(rot.get("dims", 0) or 0), float(rot.get("base", 10000.0))


class VerozenGatedLinearAttention(nn.Module):
    def __init__(self, hidden: int, mx: dict, eps: float, layer_id: int, dtype, device, low_rank: int):
        super().__init__()
        H, d, dv = mx["heads"], mx["dim"], mx["vdim"]
        self.H, self.d, self.dv, self.r = H, d, dv, low_rank
        # [q | k | v | g | a1]: every projection of the mixer's input in one GEMM
        self.in_proj = ReplicatedLinear(hidden, 2 * H * d + 2 * H * dv + low_rank, dtype, device)
        self.a2 = ReplicatedLinear(low_rank, H * d, dtype, device)
        self.a2_bias = nn.Parameter(torch.zeros(H * d, dtype=dtype, device=device), requires_grad=False)
        self.recurrence = LinearRecurrence(H, d, dv, layer_id, device, q_scale=d ** -0.5, tau=mx["tau"])
        self.norm_gate = HeadNormGate(dv, eps, dtype, device, with_weight=True)
        self.o_proj = ReplicatedLinear(H * dv, hidden, dtype, device)

    def forward(self, positions, h, forward_batch):
        T, H, d, dv = h.shape[0], self.H, self.d, self.dv
        p = self.in_proj(h)[0]
        q = p[:, : H * d].view(T, H, d)
        k = p[:, H * d: 2 * H * d].view(T, H, d)
        v = p[:, 2 * H * d: 2 * H * d + H * dv].view(T, H, dv)
        g = p[:, 2 * H * d + H * dv: 2 * H * d + 2 * H * dv]
        a1 = p[:, 2 * H * d + 2 * H * dv:]
        z = get_ops().linear(a1, self.a2.weight.data, out_dtype=torch.float32)      # gate logits, fp32 from here on
        o = self.recurrence(q, k, v, forward_batch, gate_logits=z, gate_bias=self.a2_bias.data)
        return self.o_proj(self.norm_gate(o, g))[0]


class VerozenRetention(nn.Module):
    def __init__(self, hidden: int, mx: dict, eps: float, layer_id: int, dtype, device):
        super().__init__()
        H, d, dv = mx["heads"], mx["dim"], mx["vdim"]
        self.H, self.d, self.dv = H, d, dv
        rot_dims, rot_base = _rot(mx)
        self.in_proj = ReplicatedLinear(hidden, 2 * H * d + 2 * H * dv, dtype, device)     # [q | k | v | g]
        self.q_rope = HeadNormRope(d, rot_dims, rot_base, False, eps, dtype, device, with_norm=False)
        self.k_rope = HeadNormRope(d, rot_dims, rot_base, False, eps, dtype, device, with_norm=False, scale=d ** -0.5)
        self.recurrence = LinearRecurrence(H, d, dv, layer_id, device, head_decay=mx["decay"])
        self.norm_gate = HeadNormGate(dv, eps, dtype, device, with_weight=False)
        self.o_proj = ReplicatedLinear(H * dv, hidden, dtype, device)

    def forward(self, positions, h, forward_batch):
        T, H, d, dv = h.shape[0], self.H, self.d, self.dv
        p = self.in_proj(h)[0]
        # what enters the recurrence is fp32 from the rotation on
        q = self.q_rope(p[:, : H * d].view(T, H, d), positions, torch.float32)
        k = self.k_rope(p[:, H * d: 2 * H * d].view(T, H, d), positions, torch.float32)
        v = p[:, 2 * H * d: 2 * H * d + H * dv].view(T, H, dv)
        g = p[:, 2 * H * d + H * dv:]
        o = self.recurrence(q, k, v, forward_batch)
        return self.o_proj(self.norm_gate(o, g))[0]


class VerozenSigmoidAttention(nn.Module):
    def __init__(self, hidden: int, mx: dict, eps: float, layer_id: int, dtype, device):
        super().__init__()
        H, G, d = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"]
        self.H, self.G, self.d = H, G, d
        rot_dims, rot_base = _rot(mx)
        self.in_proj = ReplicatedLinear(hidden, (H + G) * d, dtype, device)                # [q | k]
        self.q_norm = HeadNormRope(d, rot_dims, rot_base, True, eps, dtype, device, with_norm=True)
        self.k_norm = HeadNormRope(d, rot_dims, rot_base, True, eps, dtype, device, with_norm=True)
        self.raw = HeadNormRope(d, 0, 1.0, True, eps, dtype, device, with_norm=False)       # the values: keys as projected
        self.attn = SigmoidAttention(H, G, d, d, mx["scale"], layer_id, device)
        self.o_proj = ReplicatedLinear(H * d, hidden, dtype, device)

    def forward(self, positions, h, forward_batch):
        T, H, G, d = h.shape[0], self.H, self.G, self.d
        p = self.in_proj(h)[0]
        k_cache, v_cache = forward_batch.token_to_kv_pool.get_kv_buffer(self.attn.layer_id)
        k = p[:, H * d:].view(T, G, d)
        q = self.q_norm(p[:, : H * d].view(T, H, d), positions, h.dtype)
        self.k_norm(k, positions, h.dtype, cache=k_cache, loc=forward_batch.out_cache_loc)
        self.raw(k, positions, h.dtype, cache=v_cache, loc=forward_batch.out_cache_loc)
        o = torch.empty((T, H, d), dtype=h.dtype, device=h.device)
        self.attn(q, forward_batch, o)
        return self.o_proj(o.view(T, H * d))[0]


class VerozenMoE(nn.Module):
    def __init__(self, hidden: int, mlp: dict, dtype, device):
        super().__init__()
        r = mlp["router"]
        groups = r.get("groups") or {"count": 1, "keep": 1}
        self.router = GroupedTopKRouter(hidden, r["experts"], r["top"], groups["count"], groups["keep"], r.get("scale", 1.0), device)
        self.experts = GroupedExperts(hidden, mlp["expert"]["ff"], r["experts"], dtype, device)

    def forward(self, x, h):
        """x: the fp32 stream (the router reads it), h: its activation-dtype copy (the experts read it)."""
        ids, weights = self.router(x)
        y, rows = self.experts(h, ids)
        return y, rows, weights


class VerozenTokenSide(nn.Module):
    """x += RMSnorm(proj(gelu_tanh(gate x) * table[token, layer slice])) * w."""

    def __init__(self, hidden: int, dim: int, layer_id: int, eps: float, dtype, device):
        super().__init__()
        self.dim, self.layer_id = dim, layer_id
        self.gate = ReplicatedLinear(hidden, dim, dtype, device)
        self.proj = ReplicatedLinear(dim, hidden, dtype, device)
        self.add = NormedResidualAdd(hidden, eps, dtype, device)

    def forward(self, x, h, input_ids, table):
        g = get_ops().gelu_tanh_mul_rows(self.gate(h)[0], table, input_ids, self.layer_id * self.dim)
        return self.add(x, self.proj(g)[0])


class VerozenDecoderLayer(nn.Module):
    def __init__(self, config, layer_id: int, dtype, device, has_norm2: bool, gate_rank: int):
        super().__init__()
        spec = config.layer_specs[layer_id]
        D, eps = config.hidden_size, config.rms_norm_eps
        kind = spec["type"]
        if kind == "gla":
            self.mixer = VerozenGatedLinearAttention(D, spec["mixer"], eps, layer_id, dtype, device, gate_rank)
        elif kind == "retention":
            self.mixer = VerozenRetention(D, spec["mixer"], eps, layer_id, dtype, device)
        else:
            self.mixer = VerozenSigmoidAttention(D, spec["mixer"], eps, layer_id, dtype, device)
        self.norm1 = GroupRMSNorm(D, config.norm_groups, eps, dtype, device, residual_scale=config.postln_alpha)
        self.moe = VerozenMoE(D, spec["mlp"], dtype, device) if spec.get("mlp") is not None else None
        self.norm2 = (GroupRMSNorm(D, config.norm_groups, eps, dtype, device, residual_scale=config.postln_alpha)
                      if (self.moe is not None or has_norm2) else None)
        self.side = (VerozenTokenSide(D, config.token_side_dim, layer_id, eps, dtype, device)
                     if config.token_side_dim else None)

    def forward(self, positions, x, h, input_ids, side_table, forward_batch):
        h = self.norm1(x, self.mixer(positions, h, forward_batch))
        if self.moe is not None:
            y, rows, weights = self.moe(x, h)
            h = self.norm2(x, y, rows=rows, coef=weights)
        elif self.norm2 is not None:
            h = self.norm2(x)
        if self.side is not None:
            h = self.side(x, h, input_ids, side_table)
        return h


class VerozenModel(nn.Module):
    def __init__(self, config, dtype, device, norm2_layers=(), gate_ranks=None):
        super().__init__()
        D = config.hidden_size
        self.embed = nn.Parameter(torch.zeros(config.vocab_size, D, dtype=dtype, device=device), requires_grad=False)
        side = config.token_side_dim * config.num_hidden_layers
        self.side_embed = (nn.Parameter(torch.zeros(config.vocab_size, side, dtype=dtype, device=device), requires_grad=False)
                           if side else None)
        self.layers = nn.ModuleList([VerozenDecoderLayer(config, i, dtype, device, i in norm2_layers, (gate_ranks or {}).get(i, DEFAULT_GATE_RANK))
                                     for i in range(config.num_hidden_layers)])
        self.norm = GroupRMSNorm(D, config.norm_groups, config.rms_norm_eps, dtype, device)
        self.capture_streams = None     # a list here receives the fp32 residual after every layer (tests, debugging)

    def forward(self, input_ids, positions, forward_batch):
        h = get_ops().embedding(input_ids, self.embed.data)
        x = h.float()
        table = self.side_embed.data if self.side_embed is not None else None
        for layer in self.layers:
            h = layer(positions, x, h, input_ids, table, forward_batch)
            if self.capture_streams is not None:
                self.capture_streams.append(x.clone())
        return self.norm.normed(x)


class VerozenForCausalLM(nn.Module):
    needs_sequence_state = True
    supports_hip_graph = False    # a captured decode step pads the batch with row 0 of the request table, whose state slot it would overwrite

    def __init__(self, config, dtype=torch.bfloat16, device="cuda", quant_method_factory=None):
        super().__init__()
        if quant_method_factory is not None:
            raise NotImplementedError("Verozen runs unquantised (its norms, router, decays and residual are fp32 by design)")
        if get_tensor_model_parallel_world_size() != 1:
            raise NotImplementedError("Verozen: tensor parallelism is not implemented")
        self.config = config
        self.dtype = dtype
        # built by load_weights / init_random_weights: the rank of a gated-linear-attention layer's decay projection, and
        # whether a layer without feed-forward still has its second norm, are read off the checkpoint's tensors
        self.model = None
        self._device = device
        self.lm_head = ParallelLMHead(config.vocab_size, config.hidden_size, dtype, device)
        self.logits_processor = LogitsProcessor(config)

    def _build(self, norm2_layers=(), gate_ranks=None):
        self.model = VerozenModel(self.config, self.dtype, self._device, norm2_layers, gate_ranks)
        self.to(self._device)

    def sequence_state_spec(self) -> dict:
        shapes = self.config.recurrent_layer_shapes
        return dict(layer_num=0, hidden=self.config.hidden_size,
                    matrices={i: s for i, s in enumerate(shapes) if s is not None})

    @torch.no_grad()
    def forward(self, input_ids, positions, forward_batch):
        hidden_states = self.model(input_ids, positions, forward_batch)
        return self.logits_processor(input_ids, hidden_states, self.lm_head, forward_batch)

    def _linears(self):
        for layer in self.model.layers:
            mx = layer.mixer
            yield from (mx.in_proj, mx.o_proj)
            if hasattr(mx, "a2"):
                yield mx.a2
            if layer.side is not None:
                yield from (layer.side.gate, layer.side.proj)

    @torch.no_grad()
    def load_weights(self, weights: Dict[str, torch.Tensor]) -> None:
        """Checkpoint names: embed, side.embed, l<i>.norm1, l<i>.norm2, l<i>.mix.{q, k, v, g, o, norm, a1, a2, a2.b} (gla),
        l<i>.mix.{q, k, q.norm, k.norm, temp, pb, o} (attention), l<i>.mix.{q, k, v, g, o} (retention),
        l<i>.mlp.{router, correction, e<j>.up, e<j>.down}, l<i>.side.{gate, proj, norm}, final.norm, head; linear weights
        [out, in].  Projections that read the same rows are stacked, the experts' weights are stacked per layer."""
        cfg = self.config
        self._build(norm2_layers={i for i in range(cfg.num_hidden_layers) if f"l{i}.norm2" in weights},
                    gate_ranks={i: int(weights[f"l{i}.mix.a1"].shape[0]) for i, spec in enumerate(cfg.layer_specs)
                                if spec["type"] == "gla"})

        def put(param, value):
            assert tuple(param.shape) == tuple(value.shape), f"shape {tuple(value.shape)} for a parameter {tuple(param.shape)}"
            param.data.copy_(value.to(dtype=param.dtype), non_blocking=True)

        m = self.model
        put(m.embed, weights["embed"])
        if m.side_embed is not None:
            put(m.side_embed, weights["side.embed"])
        put(m.norm.weight, weights["final.norm"])
        put(self.lm_head.weight, weights["head"])
        for i, layer in enumerate(m.layers):
            p, mx, kind = f"l{i}.", layer.mixer, cfg.layer_specs[i]["type"]
            put(layer.norm1.weight, weights[p + "norm1"])
            if layer.norm2 is not None:
                put(layer.norm2.weight, weights[p + "norm2"])
            if kind == "gla":
                put(mx.in_proj.weight, torch.cat([weights[p + "mix." + n] for n in ("q", "k", "v", "g", "a1")], 0))
                put(mx.a2.weight, weights[p + "mix.a2"])
                put(mx.a2_bias, weights[p + "mix.a2.b"])
                put(mx.norm_gate.weight, weights[p + "mix.norm"])
            elif kind == "retention":
                put(mx.in_proj.weight, torch.cat([weights[p + "mix." + n] for n in ("q", "k", "v", "g")], 0))
            else:
                put(mx.in_proj.weight, torch.cat([weights[p + "mix.q"], weights[p + "mix.k"]], 0))
                put(mx.q_norm.weight, weights[p + "mix.q.norm"])
                put(mx.k_norm.weight, weights[p + "mix.k.norm"])
                put(mx.attn.temp, weights[p + "mix.temp"])
                put(mx.attn.bias, weights[p + "mix.pb"])
            put(mx.o_proj.weight, weights[p + "mix.o"])
            if layer.moe is not None:
                E = layer.moe.router.num_experts
                put(layer.moe.router.weight, weights[p + "mlp.router"])
                put(layer.moe.router.correction, weights[p + "mlp.correction"])
                put(layer.moe.experts.w_up, torch.stack([weights[f"{p}mlp.e{e}.up"] for e in range(E)]))
                put(layer.moe.experts.w_down, torch.stack([weights[f"{p}mlp.e{e}.down"] for e in range(E)]))
            if layer.side is not None:
                put(layer.side.gate.weight, weights[p + "side.gate"])
                put(layer.side.proj.weight, weights[p + "side.proj"])
                put(layer.side.add.weight, weights[p + "side.norm"])
        self.process_weights_after_loading()

    def process_weights_after_loading(self) -> None:
        for lin in self._linears():
            lin.quant_method.process_weights_after_loading(lin)

    @torch.no_grad()
    def init_random_weights(self, seed: int = 0, std: float = 0.02) -> None:
        if self.model is None:
            # without a checkpoint the decay projection's rank is the configuration's optional "gate_rank", or the default
            self._build(norm2_layers=(), gate_ranks={i: int(spec["mixer"]["gate_rank"]) for i, spec in enumerate(self.config.layer_specs)
                                                     if spec["type"] == "gla" and spec["mixer"].get("gate_rank")})
        dev = self.lm_head.weight.device
        g = torch.Generator(device=dev).manual_seed(seed)
        for name, p in self.named_parameters():
            w = torch.randn(p.shape, generator=g, device=p.device, dtype=torch.float32)
            if name.endswith("norm1.weight") or name.endswith("norm2.weight") or name.endswith("norm.weight") \
                    or name.endswith("norm_gate.weight") or name.endswith("add.weight"):
                p.data.copy_((1.0 + 0.1 * w).to(p.dtype))
            elif name.endswith("attn.temp"):
                p.data.copy_((1.0 + 0.1 * w).to(p.dtype))
            elif name.endswith("attn.bias"):
                p.data.copy_((-4.0 + 0.5 * w).to(p.dtype))
            elif name.endswith("correction") or name.endswith("a2_bias"):
                p.data.copy_((0.1 * w).to(p.dtype))
            elif name.endswith("embed") or name.endswith("side_embed"):
                p.data.copy_(w.to(p.dtype))
            else:
                p.data.copy_((w * (std if p.dim() < 2 else p.shape[-1] ** -0.5)).to(p.dtype))
        self.process_weights_after_loading()
