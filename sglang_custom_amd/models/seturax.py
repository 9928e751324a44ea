"""Seturax: a decoder-only model on an fp32 residual stream whose layers run their mixer and their feed-forward in
parallel off one norm, with a token shift in front of the mixer, sigmoid-gated residual branches, a hashed-bigram
embedding, and sliding-window multi-head latent attention with a softmax sink.  (No counterpart in the reference; the
module layout follows its model files, python/sglang/srt/models/deepseek_v2.py for the latent attention.)

Per layer (T tokens, width D), eleven launches besides the GEMMs' own:

  ShiftedLayerNorm      h = LN(x) * w,  hs = h + (h_prev - h) * mu                          1 launch, fp32 math
  a_proj(hs)            [q latent | kv latent | rope key | head-gate logits]                 1 GEMM (three projections merged)
  h_proj(h)             [ff gate | ff up | residual-gate logits 1 | 2]                       1 GEMM (four projections merged)
  latent_norms_rope_write   both latent RMS norms, rope of the shared key, cache row write   1 launch
  uq(c_q)               per-head queries [nope | rope]                                       1 GEMM
  q_nope W_uk           absorbed queries, rank wide                                          1 batched GEMM
  LatentWindowAttention rope of q inside; window, sink, head gate                            1 launch
  o_lat W_uv, o         values from the latent, output projection                            1 batched GEMM + 1 GEMM
  gelu_tanh(gate) * up, down                                                                 1 launch + 1 GEMM
  GatedResidual         x += sig(g1 + b1) * mixer + sig(g2 + b2) * ff                        1 launch, fp32

Norms, rotation angles, attention scores / weights, gates and the residual sum are fp32 in every dtype; `dtype` is what
the projections read and write.  Every size comes from the configuration, layer by layer.  Tensor parallelism is not
implemented for this family (its head counts need not divide)."""
from typing import Dict

import torch
from torch import nn

from ..distributed.parallel_state import get_tensor_model_parallel_world_size
from ..layers.activation import GeluTanhAndMul
from ..layers.latent_window_attention import LatentWindowAttention
from ..layers.linear import ReplicatedLinear
from ..layers.logits_processor import LogitsProcessor
from ..layers.token_shift import BigramHashEmbedding, GatedResidual, ShiftedLayerNorm
from ..layers.vocab_parallel_embedding import ParallelLMHead
from ..ops_backend import get_ops


class SeturaxLatentAttention(nn.Module):
    def __init__(self, hidden: int, mx: dict, eps: float, layer_id: int, dtype, device):
        super().__init__()
        self.num_heads, self.qk_nope, self.rope_dim = mx["heads"], mx["dim"], mx["rot_dim"]
        self.v_dim, self.kv_rank, self.q_rank = mx["vdim"], mx["kv_rank"], mx["q_rank"]
        self.eps = float(eps)
        H = self.num_heads
        # [dq | dkv (latent + rope key) | head gate]: three projections of the shifted rows in one GEMM
        self.a_proj = ReplicatedLinear(hidden, self.q_rank + self.kv_rank + self.rope_dim + H, dtype, device)
        self.q_norm = nn.Parameter(torch.ones(self.q_rank, dtype=dtype, device=device), requires_grad=False)
        self.kv_norm = nn.Parameter(torch.ones(self.kv_rank, dtype=dtype, device=device), requires_grad=False)
        self.uq = ReplicatedLinear(self.q_rank, H * (self.qk_nope + self.rope_dim), dtype, device)
        # per-head expansions of the latent in the layouts the absorbed form multiplies with
        self.w_uk = nn.Parameter(torch.zeros(H, self.qk_nope, self.kv_rank, dtype=dtype, device=device), requires_grad=False)
        self.w_uv = nn.Parameter(torch.zeros(H, self.kv_rank, self.v_dim, dtype=dtype, device=device), requires_grad=False)
        self.o_proj = ReplicatedLinear(H * self.v_dim, hidden, dtype, device)
        rot = mx.get("rot") or {"dims": 0, "base": 10000.0}
        self.attn = LatentWindowAttention(H, self.kv_rank, self.rope_dim, mx["scale"], mx["mask"]["size"], layer_id,
                                          rot_dims=rot["dims"], rot_base=rot["base"], device=device)

    def forward(self, positions, hs, forward_batch):
        ops = get_ops()
        T, H = hs.shape[0], self.num_heads
        a = self.a_proj(hs)[0]
        cache = forward_batch.token_to_kv_pool.get_key_buffer(self.attn.layer_id)
        cq = ops.latent_norms_rope_write(a, self.q_norm.data, self.kv_norm.data, positions, forward_batch.out_cache_loc,
                                         self.attn.inv_freq, cache, self.q_rank, self.kv_rank, self.rope_dim,
                                         self.attn.rot_dims, self.eps)
        q = self.uq(cq)[0].view(T, H, self.qk_nope + self.rope_dim)
        qa = torch.bmm(q[..., : self.qk_nope].transpose(0, 1), self.w_uk.data)             # [H, T, rank]
        gate = a[:, self.q_rank + self.kv_rank + self.rope_dim:]
        o_lat = torch.empty((H, T, self.kv_rank), dtype=hs.dtype, device=hs.device)
        self.attn(qa.transpose(0, 1), q[..., self.qk_nope:], gate, forward_batch, o_lat.transpose(0, 1))
        o = torch.bmm(o_lat, self.w_uv.data)                                                # [H, T, v]
        return self.o_proj(o.transpose(0, 1).reshape(T, H * self.v_dim))[0]


class SeturaxDecoderLayer(nn.Module):
    def __init__(self, config, layer_id: int, dtype, device):
        super().__init__()
        spec = config.layer_specs[layer_id]
        D = config.hidden_size
        self.hidden = D
        self.norm1 = ShiftedLayerNorm(D, config.rms_norm_eps, dtype, device, state_layer=layer_id)
        self.mixer = SeturaxLatentAttention(D, spec["mixer"], config.rms_norm_eps, layer_id, dtype, device)
        self.ff = spec["mlp"]["ff"] if spec.get("mlp") is not None else 0
        # [ff gate | ff up | residual gate of the mixer | of the feed-forward]: every projection of the unshifted rows
        self.h_proj = ReplicatedLinear(D, 2 * self.ff + (2 if self.ff else 1) * D, dtype, device)
        self.down_proj = ReplicatedLinear(self.ff, D, dtype, device) if self.ff else None
        self.act_fn = GeluTanhAndMul()
        self.gated = GatedResidual(D, dtype, device, branches=2 if self.ff else 1)

    def forward(self, positions, x, forward_batch):
        h, hs = self.norm1(x, positions, forward_batch)
        mix = self.mixer(positions, hs, forward_batch)
        hp = self.h_proj(h)[0]
        ff, D = self.ff, self.hidden
        if ff:
            y = self.down_proj(self.act_fn(hp[:, :ff], hp[:, ff: 2 * ff]))[0]
            return self.gated(x, hp[:, 2 * ff: 2 * ff + D], mix, hp[:, 2 * ff + D:], y)
        return self.gated(x, hp[:, :D], mix)


class SeturaxModel(nn.Module):
    def __init__(self, config, dtype, device):
        super().__init__()
        bg = config.bigram
        self.embed = BigramHashEmbedding(config.vocab_size, config.hidden_size, config.embedding_scale, bg["buckets"],
                                         bg["mul_prev"], bg["mul_cur"], dtype, device)
        self.layers = nn.ModuleList([SeturaxDecoderLayer(config, i, dtype, device) for i in range(config.num_hidden_layers)])
        self.norm = ShiftedLayerNorm(config.hidden_size, config.rms_norm_eps, dtype, device)
        self.capture_streams = None     # a list here receives the fp32 residual after every layer (tests, debugging)

    def forward(self, input_ids, positions, forward_batch):
        x = self.embed(input_ids, positions, forward_batch)
        for layer in self.layers:
            x = layer(positions, x, forward_batch)
            if self.capture_streams is not None:
                self.capture_streams.append(x.clone())
        forward_batch.seq_state.commit(input_ids)     # every reader of the old state has run
        return self.norm(x)


class SeturaxForCausalLM(nn.Module):
    needs_sequence_state = True
    supports_hip_graph = False    # a captured decode step pads the batch with row 0 of the request table, whose state slot it would overwrite

    def __init__(self, config, dtype=torch.bfloat16, device="cuda", quant_method_factory=None):
        super().__init__()
        if quant_method_factory is not None:
            raise NotImplementedError("Seturax runs unquantised (its norms, gates and residual are fp32 by design)")
        if get_tensor_model_parallel_world_size() != 1:
            raise NotImplementedError("Seturax: tensor parallelism is not implemented")
        self.config = config
        self.dtype = dtype
        self.model = SeturaxModel(config, dtype, device)
        self.lm_head = ParallelLMHead(config.vocab_size, config.hidden_size, dtype, device)
        self.logits_processor = LogitsProcessor(config, logit_scale=config.logit_scale)
        self.to(device)

    def sequence_state_spec(self) -> dict:
        return dict(layer_num=self.config.num_hidden_layers, hidden=self.config.hidden_size)

    @torch.no_grad()
    def forward(self, input_ids, positions, forward_batch):
        hidden_states = self.model(input_ids, positions, forward_batch)
        return self.logits_processor(input_ids, hidden_states, self.lm_head, forward_batch)

    def _linears(self):
        for layer in self.model.layers:
            yield from (layer.mixer.a_proj, layer.mixer.uq, layer.mixer.o_proj, layer.h_proj)
            if layer.down_proj is not None:
                yield layer.down_proj

    @torch.no_grad()
    def load_weights(self, weights: Dict[str, torch.Tensor]) -> None:
        """Checkpoint names: embed, bigram, l<i>.norm1, l<i>.shift, l<i>.rg1(.b), l<i>.rg2(.b), l<i>.mix.{dq, dq.norm, uq, dkv,
        dkv.norm, uk, uv, sink, g, o}, l<i>.mlp.{gate, up, down}, final.norm, head; linear weights [out, in].  Projections
        that read the same rows are stacked (dq | dkv | g, and gate | up | rg1 | rg2), uk / uv are split per head."""
        def put(param, value):
            assert tuple(param.shape) == tuple(value.shape), f"shape {tuple(value.shape)} for a parameter {tuple(param.shape)}"
            param.data.copy_(value.to(dtype=param.dtype), non_blocking=True)

        m = self.model
        put(m.embed.weight, weights["embed"])
        put(m.embed.bigram, weights["bigram"])
        put(m.norm.weight, weights["final.norm"])
        put(self.lm_head.weight, weights["head"])
        for i, layer in enumerate(m.layers):
            p, mx = f"l{i}.", layer.mixer
            put(layer.norm1.weight, weights[p + "norm1"])
            put(layer.norm1.shift, weights[p + "shift"])
            put(mx.a_proj.weight, torch.cat([weights[p + "mix.dq"], weights[p + "mix.dkv"], weights[p + "mix.g"]], 0))
            put(mx.q_norm, weights[p + "mix.dq.norm"])
            put(mx.kv_norm, weights[p + "mix.dkv.norm"])
            put(mx.uq.weight, weights[p + "mix.uq"])
            put(mx.w_uk, weights[p + "mix.uk"].view(mx.num_heads, mx.qk_nope, mx.kv_rank))
            put(mx.w_uv, weights[p + "mix.uv"].view(mx.num_heads, mx.v_dim, mx.kv_rank).transpose(1, 2))
            put(mx.attn.sink, weights[p + "mix.sink"])
            put(mx.o_proj.weight, weights[p + "mix.o"])
            put(layer.gated.bias1, weights[p + "rg1.b"])
            if layer.ff:
                put(layer.h_proj.weight, torch.cat([weights[p + "mlp.gate"], weights[p + "mlp.up"], weights[p + "rg1"],
                                                    weights[p + "rg2"]], 0))
                put(layer.gated.bias2, weights[p + "rg2.b"])
                put(layer.down_proj.weight, weights[p + "mlp.down"])
            else:
                put(layer.h_proj.weight, weights[p + "rg1"])
        self.process_weights_after_loading()

    def process_weights_after_loading(self) -> None:
        for lin in self._linears():
            lin.quant_method.process_weights_after_loading(lin)

    @torch.no_grad()
    def init_random_weights(self, seed: int = 0, std: float = 0.02) -> None:
        dev = self.lm_head.weight.device
        g = torch.Generator(device=dev).manual_seed(seed)
        for name, p in self.named_parameters():
            w = torch.randn(p.shape, generator=g, device=p.device, dtype=torch.float32)
            if name.endswith("norm.weight") or name.endswith("norm1.weight") or name.endswith("q_norm") or name.endswith("kv_norm"):
                p.data.copy_((1.0 + 0.1 * w).to(p.dtype))
            elif name.endswith("shift"):
                p.data.copy_(torch.sigmoid(w).to(p.dtype))
            elif name.endswith("embed.weight"):
                p.data.copy_((w / self.model.embed.scale).to(p.dtype))
            elif name.endswith("bigram") or name.endswith("sink"):
                p.data.copy_((0.5 * w).to(p.dtype))
            else:
                p.data.copy_((w * (std if p.dim() < 2 else p.shape[-1] ** -0.5)).to(p.dtype))
        self.process_weights_after_loading()
