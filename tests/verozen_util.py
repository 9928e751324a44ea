"""Shared pieces of the Verozen tests: small random models in checkpoint form and the replay of a schedule with every
logit compared against the whole-sequence oracle (oracle/verozen_ref.py)."""
import torch

from oracle import verozen_ref as ref
from seturax_util import build_runner, pools_are_whole, random_prompts, rel_err  # noqa: F401  (generic helpers)


def gla(heads=3, dim=8, vdim=12, tau=4.0, rank=5):
    return dict(type="gla", mixer=dict(heads=heads, dim=dim, vdim=vdim, tau=tau), _rank=rank)


def attention(heads=4, kv_heads=2, dim=16, rot_dims=8, base=100.0, scale=0.3):
    return dict(type="attention", mixer=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=scale,
                                             rot=dict(dims=rot_dims, base=base)))


def retention(heads=2, dim=12, vdim=20, rot_dims=12, base=50.0, decay=(0.9, 0.97)):
    return dict(type="retention", mixer=dict(heads=heads, dim=dim, vdim=vdim, decay=list(decay), rot=dict(dims=rot_dims, base=base)))


def moe(experts=6, top=2, count=3, keep=2, ff=20, scale=1.25):
    return dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top, scale=scale, groups=dict(count=count, keep=keep)))


def make_config(layers=None, width=48, vocab=53, groups=3, alpha=2.0, side=6, eps=1e-5):
    """layers: list of (mixer spec, mlp spec or None).  The default stacks the three mixers with unlike sizes."""
    if layers is None:
        layers = [(gla(), moe()), (attention(), moe(experts=4, top=3, count=1, keep=1)), (retention(), None),
                  (gla(heads=1, dim=20, vdim=4, tau=1.0, rank=3), moe(experts=8, top=1, count=8, keep=3))]
    cfg = dict(architecture="Verozen", vocab=vocab, width=width, postln_alpha=alpha, norm=dict(eps=eps, groups=groups),
               layers=[dict(type=m["type"], mixer=dict(m["mixer"]), mlp=f) for m, f in layers])
    if side:
        cfg["token_side"] = dict(dim=side)
    cfg["_ranks"] = [m.get("_rank") for m, _ in layers]      # read by make_weights only
    return cfg


def make_weights(cfg, seed=0, norm2_without_mlp=False, separated_router=False):
    """Checkpoint-named tensors with bf16-representable values, so that a bf16 and an fp32 run read the same numbers.
    separated_router: the selection corrections lie 1.5 apart in a shuffled order, so that no rounding of the scores (which
    lie in (0, 1)) can change which experts are chosen -- a bf16 run against a float64 oracle would otherwise rest on close
    calls; the experts' weights still depend on the token."""
    g = torch.Generator().manual_seed(seed)
    D, V, L = cfg["width"], cfg["vocab"], len(cfg["layers"])

    def rnd(*shape, std=1.0, mean=0.0):
        return (mean + std * torch.randn(*shape, generator=g)).to(torch.bfloat16)

    w = {"embed": rnd(V, D), "final.norm": rnd(D, std=0.1, mean=1.0), "head": rnd(V, D, std=D ** -0.5)}
    side = (cfg.get("token_side") or {}).get("dim", 0)
    if side:
        w["side.embed"] = rnd(V, L * side)
    for i, spec in enumerate(cfg["layers"]):
        p, m, kind = f"l{i}.", spec["mixer"], spec["type"]
        H, d = m["heads"], m["dim"]
        w[p + "norm1"] = rnd(D, std=0.1, mean=1.0)
        if kind == "attention":
            G = m.get("kv_heads", H)
            w[p + "mix.q"], w[p + "mix.k"] = rnd(H * d, D, std=D ** -0.5), rnd(G * d, D, std=D ** -0.5)
            w[p + "mix.q.norm"], w[p + "mix.k.norm"] = rnd(d, std=0.1, mean=1.0), rnd(d, std=0.1, mean=1.0)
            w[p + "mix.temp"], w[p + "mix.pb"] = rnd(H, std=0.2, mean=1.0), rnd(H, std=0.5, mean=-2.0)
            w[p + "mix.o"] = rnd(D, H * d, std=(H * d) ** -0.5)
        else:
            dv = m["vdim"]
            for n, rows in (("q", H * d), ("k", H * d), ("v", H * dv), ("g", H * dv)):
                w[p + "mix." + n] = rnd(rows, D, std=D ** -0.5)
            w[p + "mix.o"] = rnd(D, H * dv, std=(H * dv) ** -0.5)
            if kind == "gla":
                r = cfg["_ranks"][i] or 4
                w[p + "mix.norm"] = rnd(dv, std=0.1, mean=1.0)
                w[p + "mix.a1"], w[p + "mix.a2"] = rnd(r, D, std=D ** -0.5), rnd(H * d, r, std=2.0 * r ** -0.5)
                w[p + "mix.a2.b"] = rnd(H * d, std=1.0, mean=1.0)
        if spec["mlp"] is not None:
            ff, E = spec["mlp"]["expert"]["ff"], spec["mlp"]["router"]["experts"]
            w[p + "norm2"] = rnd(D, std=0.1, mean=1.0)
            w[p + "mlp.router"] = rnd(E, D, std=2.0 * D ** -0.5)
            w[p + "mlp.correction"] = rnd(E, std=0.5, mean=-0.5)        # selection scores of both signs
            if separated_router:
                w[p + "mlp.correction"] = ((torch.randperm(E, generator=g).float() - E / 2) * 1.5).to(torch.bfloat16)
            for e in range(E):
                w[f"{p}mlp.e{e}.up"], w[f"{p}mlp.e{e}.down"] = rnd(ff, D, std=D ** -0.5), rnd(D, ff, std=ff ** -0.5)
        elif norm2_without_mlp:
            w[p + "norm2"] = rnd(D, std=0.1, mean=1.0)
        if side:
            w[p + "side.gate"], w[p + "side.proj"] = rnd(side, D, std=D ** -0.5), rnd(D, side, std=side ** -0.5)
            w[p + "side.norm"] = rnd(D, std=0.1, mean=0.5)
    return w


def public(cfg):
    """The configuration as a model folder would hold it (without the helper entries of make_config)."""
    return {k: v for k, v in cfg.items() if not k.startswith("_")}


def replay_and_compare(runner, cfg, weights, prompts, schedule, tol):
    """schedule: list of steps, each a list of (request name, token count).  Every token's logits are asked for and
    compared with the oracle's logits of the whole prompt; a request ends with its last token.  Returns the worst error."""
    from sglang_custom_amd.managers.trace_replay import TraceReplayer

    rp = TraceReplayer(runner)
    want = {k: ref.forward(public(cfg), weights, p) for k, p in prompts.items()}
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
