"""Shared pieces of the Seturax tests: small random models in checkpoint form, a runner on either device, and the
replay of a schedule with every logit compared against the whole-sequence oracle (oracle/seturax_ref.py)."""
import math

import torch

from oracle import seturax_ref as ref


def mixer(heads, dim, rot_dim, vdim, kv_rank, q_rank, window, base=10000.0, scale=None):
    return dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, q_rank=q_rank, mask=dict(size=window),
                rot=dict(base=base, dims=rot_dim), scale=scale if scale is not None else 1.0 / math.sqrt(dim + rot_dim))


def make_config(width=48, vocab=61, layers=None, buckets=13, mul_prev=7, mul_cur=3, scale=4.0, logit_scale=0.5, eps=1e-5):
    if layers is None:
        # three unlike layers: head counts 3 / 2 / 1, a window of 1 (sees only itself), one without feed-forward
        layers = [(mixer(3, 8, 4, 6, 10, 12, 5), 40), (mixer(2, 16, 8, 8, 24, 16, 1, base=500.0), None),
                  (mixer(1, 8, 2, 12, 16, 8, 9), 56)]
    return dict(architecture="Seturax", vocab=vocab, width=width, logit_scale=logit_scale, norm=dict(eps=eps),
                embedding=dict(scale=scale, bigram=dict(buckets=buckets, mul_prev=mul_prev, mul_cur=mul_cur)),
                layers=[dict(type="latent_attention", mixer=m, mlp=None if ff is None else dict(kind="dense", ff=ff))
                        for m, ff in layers])


def make_weights(cfg, seed=0):
    """Checkpoint-named tensors with bf16-representable values, so that a bf16 and an fp32 run read the same numbers."""
    g = torch.Generator().manual_seed(seed)
    D, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, std=1.0, mean=0.0):
        return (mean + std * torch.randn(*shape, generator=g)).to(torch.bfloat16)

    w = {"embed": rnd(V, D, std=1.0 / cfg["embedding"]["scale"]), "bigram": rnd(cfg["embedding"]["bigram"]["buckets"] + 1, D, std=0.5),
         "final.norm": rnd(D, std=0.1, mean=1.0), "head": rnd(V, D, std=D ** -0.5)}
    for i, spec in enumerate(cfg["layers"]):
        p, m = f"l{i}.", spec["mixer"]
        H, dn, dr, dv, rk, qk = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
        w[p + "norm1"] = rnd(D, std=0.1, mean=1.0)
        w[p + "shift"] = torch.rand(D, generator=g).to(torch.bfloat16)
        w[p + "mix.dq"] = rnd(qk, D, std=D ** -0.5)
        w[p + "mix.dq.norm"] = rnd(qk, std=0.1, mean=1.0)
        w[p + "mix.uq"] = rnd(H * (dn + dr), qk, std=2.0 * qk ** -0.5)
        w[p + "mix.dkv"] = rnd(rk + dr, D, std=D ** -0.5)
        w[p + "mix.dkv.norm"] = rnd(rk, std=0.1, mean=1.0)
        w[p + "mix.uk"] = rnd(H * dn, rk, std=2.0 * rk ** -0.5)
        w[p + "mix.uv"] = rnd(H * dv, rk, std=rk ** -0.5)
        w[p + "mix.sink"] = rnd(H, std=1.0)
        w[p + "mix.g"] = rnd(H, D, std=D ** -0.5)
        w[p + "mix.o"] = rnd(D, H * dv, std=(H * dv) ** -0.5)
        for r in ("rg1", "rg2"):
            w[p + r] = rnd(D, D, std=D ** -0.5)
            w[p + r + ".b"] = rnd(D, std=0.5)
        if spec["mlp"] is not None:
            ff = spec["mlp"]["ff"]
            w[p + "mlp.gate"] = rnd(ff, D, std=D ** -0.5)
            w[p + "mlp.up"] = rnd(ff, D, std=D ** -0.5)
            w[p + "mlp.down"] = rnd(D, ff, std=ff ** -0.5)
    return w


def build_runner(cfg, weights, dtype="float32", device="cpu", max_total_tokens=256, max_running_requests=4, **server_args):
    from sglang_custom_amd.configs.model_config import ModelConfig
    from sglang_custom_amd.model_executor.model_runner import ModelRunner
    from sglang_custom_amd.server_args import ServerArgs

    mc = ModelConfig(cfg, dtype=dtype, context_length=max_total_tokens)
    sa = ServerArgs(dtype=dtype, device=device, max_total_tokens=max_total_tokens, max_running_requests=max_running_requests,
                    context_length=max_total_tokens, **server_args)
    return ModelRunner(mc, sa, weights={k: v.to(device) for k, v in weights.items()})


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """Worst row of: rms over the vocabulary of the difference (means taken off) over the rms of the expected row."""
    d = got.double().cpu() - want.double()
    d = d - d.mean(-1, keepdim=True)
    w = want.double() - want.double().mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-9)).max())


def replay_and_compare(runner, cfg, weights, prompts, schedule, tol):
    """schedule: list of steps, each a list of (request name, token count).  Every token's logits are asked for and
    compared with the oracle's logits of the whole prompt; a request ends with its last token.  Returns the worst error."""
    from sglang_custom_amd.managers.trace_replay import TraceReplayer

    rp = TraceReplayer(runner)
    want = {k: ref.forward(cfg, weights, p) for k, p in prompts.items()}
    at = {k: 0 for k in prompts}
    worst = 0.0
    for step in schedule:
        entries, rows, end = [], [], []
        for name, n in step:
            lo, hi = at[name], at[name] + n
            entries.append(dict(id=name, tokens=prompts[name][lo:hi], want=list(range(n))))
            rows.append(want[name][lo:hi])
            at[name] = hi
            if hi == len(prompts[name]):
                end.append(name)
        got = rp.step(entries, end)
        e = rel_err(got, torch.cat(rows))
        assert e < tol, f"step {step}: logits differ from the whole-sequence oracle by {e:.3g} (limit {tol})"
        worst = max(worst, e)
    assert all(at[k] == len(p) for k, p in prompts.items()), "the schedule does not cover the prompts"
    assert not rp.live
    return worst


def random_prompts(cfg, lengths, seed=0):
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, cfg["vocab"], (n,), generator=g).tolist() for i, n in enumerate(lengths)}


def pools_are_whole(runner) -> bool:
    """Every KV slot, request row and state slot is back."""
    mr = runner
    return (mr.token_to_kv_pool_allocator.available_size() == mr.max_total_num_tokens
            and mr.req_to_token_pool.available_size() == mr.req_to_token_pool.size
            and mr.req_to_token_pool.state_pool.available_size() == mr.req_to_token_pool.state_pool.size)
