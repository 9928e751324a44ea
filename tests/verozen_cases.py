"""Checks of single Verozen mechanisms against the oracle's functions (oracle/verozen_ref.py), written once for any ops
object: the HIP kernels on the GPU (test_verozen_gpu.py) and the CPU stand-ins (test_verozen_cpu.py).  Every case builds
the request table, positions and state pool by hand, so that slots, pages and cuts are the case's to choose."""
import math

import torch

from oracle import verozen_ref as ref


def _dev(t, device):
    return t.to(device) if t is not None else None


def _bf(x):
    return x.to(torch.bfloat16).to(torch.float64)


def _tol(dtype):
    return 2e-5 if dtype == torch.float32 else 2e-2


def _close(got, want, tol, what):
    got, want = got.detach().cpu().double(), want.double()
    err = (got - want).abs().max() / want.abs().max().clamp_min(1e-6)
    assert float(err) < tol, f"{what}: relative error {float(err):.3g} (limit {tol})"


def check_group_norm(ops, device, dtype, T=7, D=48, groups=3, alpha=2.5, eps=1e-5):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(T, D, generator=g)
    y = _bf(torch.randn(T, D, generator=g))
    w = _bf(1 + 0.1 * torch.randn(D, generator=g))
    want = ref.group_rms_norm(alpha * x.double() + y, w, groups, eps)
    xd = x.clone().to(device)
    h = ops.scaled_add_group_rmsnorm(xd, y.to(dtype).to(device), alpha, w.to(dtype).to(device), groups, eps)
    _close(xd, want, 2e-6, "the fp32 stream after the norm")
    _close(h, want, _tol(dtype), "its activation-dtype copy")
    # the branch as a weighted sum of picked rows, and the norm alone (not in place)
    big = _bf(torch.randn(3 * T + 2, D, generator=g))
    rows = torch.randint(0, 3 * T + 2, (T, 3), generator=g, dtype=torch.int32)
    coef = torch.rand(T, 3, generator=g)
    want2 = ref.group_rms_norm(alpha * x.double() + (coef.double()[:, :, None] * big[rows.long()]).sum(1), w, groups, eps)
    xd = x.clone().to(device)
    ops.scaled_add_group_rmsnorm(xd, big.to(dtype).to(device), alpha, w.to(dtype).to(device), groups, eps, rows=rows.to(device),
                                 coef=coef.to(device))
    _close(xd, want2, 2e-6, "the norm over a weighted sum of rows")
    xd = x.clone().to(device)
    h = ops.scaled_add_group_rmsnorm(xd, None, 1.0, w.to(dtype).to(device), groups, eps, inplace=False)
    assert torch.equal(xd.cpu(), x), "a norm that is not in place leaves its input"
    _close(h, ref.group_rms_norm(x.double(), w, groups, eps), _tol(dtype), "the norm alone")
    # x += y / rms(y) * w
    xd = x.clone().to(device)
    ops.rmsnorm_residual_add(xd, y.to(dtype).to(device), w.to(dtype).to(device), eps)
    _close(xd, x.double() + ref.unit_rms(y, eps) * w, 2e-6, "the normed residual add")


# an angle of 700 radians held in fp32 (frequencies rounded to fp32, then the product) is good to about 5e-5 radians
ROT32 = 1e-4


def check_head_norm_rope(ops, device, dtype, interleaved, rot_dims, d=24, H=3, with_norm=True, scale=0.5, base=37.0, eps=1e-5):
    g = torch.Generator().manual_seed(1)
    T = 9
    src = _bf(torch.randn(T, H, d, generator=g))
    w = _bf(1 + 0.1 * torch.randn(d, generator=g)) if with_norm else None
    positions = torch.tensor([0, 1, 2, 700, 701, 5, 6, 63, 64], dtype=torch.int64)
    # the oracle rotates row p of a sequence by position p: lay the rows out at their positions
    n = int(positions.max()) + 1
    full = torch.zeros(n, H, d, dtype=torch.float64)
    full[positions] = (ref.unit_rms(src, eps) * w) if with_norm else src
    want = ref.rotate_pairs(full, rot_dims, base, interleaved)[positions] * scale
    i = torch.arange(max(rot_dims // 2, 1), dtype=torch.float64)
    inv_freq = (base ** (-2.0 * i / max(rot_dims, 1))).float().to(device)
    wide = torch.zeros(T, H * d + 5, dtype=dtype)              # rows inside a wider projection output
    wide[:, 2: 2 + H * d] = src.reshape(T, H * d).to(dtype)
    view = wide.to(device)[:, 2: 2 + H * d].view(T, H, d)
    for out_dtype in {dtype, torch.float32}:
        got = ops.head_norm_rope(view, _dev(w.to(dtype), device) if with_norm else None, eps, positions.to(device), inv_freq,
                                 rot_dims, interleaved, scale, out_dtype)
        assert got.dtype == out_dtype
        _close(got, want, _tol(dtype) if out_dtype != torch.float32 else ROT32, f"rotation, pairs {'2i,2i+1' if interleaved else 'i,i+n/2'}")
    cache = torch.zeros(40, H, d, dtype=dtype, device=device)
    loc = torch.tensor([7, 3, 39, 1, 2, 20, 21, 8, 9], dtype=torch.int64, device=device)
    ops.head_norm_rope(view, _dev(w.to(dtype), device) if with_norm else None, eps, positions.to(device), inv_freq, rot_dims,
                       interleaved, scale, dtype, cache=cache, loc=loc)
    _close(cache[loc], want, max(_tol(dtype), ROT32), "rows written into the cache")
    assert float(cache[0].abs().max()) == 0.0


class Table:
    """A request table, positions and segments for hand-made batches."""

    def __init__(self, device, rows=6, width=2048):
        self.device = device
        self.req_to_token = torch.zeros((rows, width), dtype=torch.int32, device=device)
        self.req_to_state = torch.zeros(rows, dtype=torch.int32, device=device)

    def batch(self, segs):
        """segs: list of (request row, first position, count) -> dict of device tensors."""
        rp, pos, tr, ss, sl, at = [], [], [], [], [], 0
        for b, (row, p0, n) in enumerate(segs):
            rp.append(row)
            pos += list(range(p0, p0 + n))
            tr += [b] * n
            ss.append(at)
            sl.append(n)
            at += n
        d = self.device
        return dict(req_pool_indices=torch.tensor(rp, dtype=torch.int64, device=d), positions=torch.tensor(pos, dtype=torch.int64, device=d),
                    tok_req=torch.tensor(tr, dtype=torch.int32, device=d), seg_start=torch.tensor(ss, dtype=torch.int32, device=d),
                    seg_len=torch.tensor(sl, dtype=torch.int32, device=d))


def run_recurrence(ops, device, dtype, q, k, v, cuts, log_a=None, decay=None, tau=1.0, q_scale=1.0, qk_fp32=False, slot=2, state=None,
                   decode_tail=0):
    """One sequence cut into portions (the last decode_tail tokens as decode steps without segment arrays)."""
    T, H, dk = q.shape
    dv = v.shape[-1]
    tab = Table(device)
    tab.req_to_state[4] = slot
    if state is None:
        state = torch.full((5, H, dk, dv), 77.0, dtype=torch.float32, device=device)     # stale: position 0 must not read it
    qd = q.to(torch.float32 if qk_fp32 else dtype).to(device)
    kd = k.to(torch.float32 if qk_fp32 else dtype).to(device)
    vd = v.to(dtype).to(device)
    z = bias = hd = None
    if log_a is not None:
        # logits whose logsigmoid / tau is log_a: z = log(a^tau / (1 - a^tau)); half of it goes through the bias
        p = torch.exp(log_a.double() * tau).clamp(1e-12, 1 - 1e-12)
        zz = torch.log(p / (1 - p)).reshape(T, H * dk)
        bias = _bf(0.5 * zz.mean(0))
        z = (zz - bias).float().to(device)
        bias = bias.to(dtype).to(device)
    else:
        hd = torch.tensor(list(decay), dtype=torch.float32, device=device)
    outs, at = [], 0
    for n in cuts:
        decode = at >= T - decode_tail and n == 1
        b = tab.batch([(4, at, n)])
        o = torch.empty((n, H, dv), dtype=torch.float32, device=device)
        seg = {} if decode else dict(tok_req=b["tok_req"], seg_start=b["seg_start"], seg_len=b["seg_len"])
        ops.linear_recurrence(qd[at:at + n], kd[at:at + n], vd[at:at + n], o, state, tab.req_to_state, b["req_pool_indices"],
                              b["positions"], q_scale, gate_logits=z[at:at + n] if z is not None else None, gate_bias=bias, tau=tau,
                              head_decay=hd, **seg)
        outs.append(o.cpu())
        at += n
    assert at == T
    return torch.cat(outs), state


def check_recurrence(ops, device, dtype, per_channel, H=3, dk=12, dv=20, T=45, cuts=(45,), tau=4.0, decode_tail=0):
    g = torch.Generator().manual_seed(2)
    q, k, v = (_bf(torch.randn(T, H, n, generator=g)) for n in (dk, dk, dv))
    scale = 0.37
    if per_channel:
        log_a = -torch.rand(T, H, dk, generator=g).double() * 0.5
        want = ref.decayed_sum_per_channel(q * scale, k, v, log_a)
        got, _ = run_recurrence(ops, device, dtype, q, k, v, cuts, log_a=log_a, tau=tau, q_scale=scale, decode_tail=decode_tail)
        tol = 5e-3 if dtype == torch.float32 else 2e-2        # the decays make the trip through bf16-rounded biases
    else:
        decay = [1.0, 0.5, 0.97][:H] + [0.9] * max(0, H - 3)
        want = ref.decayed_sum_per_head(q * scale, k, v, decay)
        got, _ = run_recurrence(ops, device, dtype, q, k, v, cuts, decay=decay, q_scale=scale, qk_fp32=True, decode_tail=decode_tail)
        tol = 2e-5
    _close(got, want, tol, f"recurrence cut into {list(cuts)[:6]}")


def check_recurrence_far_key(ops, device, dtype):
    """With decay 1 a key 600 tokens back is remembered in full, with decay 0.5 it is gone; the first token of a sequence
    starts from zero whatever the slot held; a portion's first token starts from what the last portion left."""
    H, dk, dv, T = 2, 8, 8, 640
    q = torch.zeros(T, H, dk, dtype=torch.float64)
    k = torch.zeros(T, H, dk, dtype=torch.float64)
    v = torch.zeros(T, H, dv, dtype=torch.float64)
    k[3, :, 1] = 1.0
    v[3, :, 5] = 2.0
    q[T - 1, :, 1] = 1.0
    q[4, :, 1] = 1.0
    for cuts in ([T], [4, 2, 600, 34], [5] + [127] * 5):
        got, state = run_recurrence(ops, device, dtype, q, k, v, cuts, decay=[1.0, 0.5], qk_fp32=True)
        assert abs(float(got[T - 1, 0, 5]) - 2.0) < 1e-6 and float(got[T - 1, 1, 5]) < 1e-30, cuts
        assert abs(float(got[4, 1, 5]) - 1.0) < 1e-6 and float(got[:3].abs().max()) == 0.0, cuts
        assert abs(float(state[2, 0, 1, 5]) - 2.0) < 1e-6 and float(state[1].min()) == 77.0, "only the sequence's slot is written"


class KVSetup:
    """Keys / values of one sequence scattered over cache slots through a request-table row."""

    def __init__(self, device, dtype, kn, v, row=3, page=1, seed=5):
        T, G, d = kn.shape
        g = torch.Generator().manual_seed(seed)
        self.tab = Table(device)
        n_slots = T + 70 if page == 1 else (T // page + 4) * page
        if page == 1:
            slots = torch.randperm(n_slots - 1, generator=g)[:T] + 1
        else:
            pages = torch.randperm((n_slots - 1) // page - 1, generator=g) + 1
            slots = (pages[:, None] * page + torch.arange(page)[None, :]).reshape(-1)[:T]
        self.k_cache = torch.zeros(n_slots + page, G, d, dtype=dtype, device=device)
        self.v_cache = torch.zeros(n_slots + page, G, v.shape[-1], dtype=dtype, device=device)
        self.k_cache[slots.to(device)] = kn.to(dtype).to(device)
        self.v_cache[slots.to(device)] = v.to(dtype).to(device)
        self.tab.req_to_token[row, :T] = slots.to(torch.int32).to(device)
        self.row = row


def run_sigmoid_attention(ops, device, dtype, q, kn, v, scale, temp, bias, cuts, page=1, decode_tail=0, splits=1):
    T, H, d = q.shape
    G = kn.shape[1]
    kv = KVSetup(device, dtype, kn, v, page=page)
    bq = ops.sigmoid_attention_block_tokens(H, G, d, v.shape[-1], dtype)
    qd = q.to(dtype).to(device)
    outs, at = [], 0
    for n in cuts:
        decode = at >= T - decode_tail and n == 1
        b = kv.tab.batch([(kv.row, at, n)])
        o = torch.zeros((n, H, v.shape[-1]), dtype=dtype, device=device)
        blocks = None
        if not decode:
            runs = [[s, min(bq, n - s)] for s in range(0, n, bq)]
            blocks = torch.tensor(runs, dtype=torch.int32, device=device)
        ops.sigmoid_attention(qd[at:at + n], kv.k_cache, kv.v_cache, o, kv.tab.req_to_token, b["req_pool_indices"], b["positions"],
                              temp.float().to(device), bias.float().to(device), scale, tok_req=None if decode else b["tok_req"],
                              blocks=blocks, num_splits=splits if decode else 1, max_run=bq)
        outs.append(o.cpu())
        at += n
    return torch.cat(outs)


def check_sigmoid_attention(ops, device, dtype, H=4, G=2, d=32, T=150, cuts=(150,), page=1, decode_tail=0, splits=1):
    g = torch.Generator().manual_seed(3)
    q = _bf(torch.randn(T, H, d, generator=g))
    kn = _bf(torch.randn(T, G, d, generator=g))
    v = _bf(torch.randn(T, G, d, generator=g))
    temp = 1 + 0.2 * torch.randn(H, generator=g).double()
    bias = -2 + 0.5 * torch.randn(H, generator=g).double()
    scale = 1.0 / math.sqrt(d)
    want = ref.sigmoid_weighted_sum(q, kn, v, scale, temp.float().double(), bias.float().double())
    got = run_sigmoid_attention(ops, device, dtype, q, kn, v, scale, temp, bias, cuts, page=page, decode_tail=decode_tail, splits=splits)
    _close(got, want, 2e-5 if dtype == torch.float32 else 1.5e-2, f"sigmoid attention cut into {list(cuts)[:6]}, pages of {page}")


def check_sigmoid_attention_planted(ops, device, dtype):
    """A bias of -30 silences every key but the ones whose score is made large: one far back among hundreds, the query's
    own key (the last one it may see), and the key right after it (which it must not see), at a page's border too."""
    H, G, d, T = 2, 1, 32, 700
    q = torch.zeros(T, H, d, dtype=torch.float64)
    kn = torch.zeros(T, G, d, dtype=torch.float64)
    v = torch.zeros(T, G, d, dtype=torch.float64)
    for j, col in ((2, 0), (63, 1), (64, 2), (65, 3), (699, 4)):
        kn[j, 0, col] = 8.0
        v[j, 0, col] = 1.0 + col
    temp, bias = torch.ones(H, dtype=torch.float64), torch.full((H,), -30.0, dtype=torch.float64)
    def ask(i, cols):
        q[i] = 0
        for c in cols:
            q[i, :, c] = 8.0
    ask(698, [0])          # far: key 2 seen from 698
    ask(63, [1, 2])        # its own key (63) is seen, the next one (64) is not
    ask(64, [2, 3])        # the same across a border of 64: 64 seen, 65 not
    ask(699, [4, 0])       # the last token sees itself and the far key
    for cuts, tail in (([T], 0), ([60, 3, 2, 635], 0), ([64, 1, 634, 1], 0), ([698, 1, 1], 2)):
        for page in (1, 64):
            got = run_sigmoid_attention(ops, device, dtype, q, kn, v, 1.0, temp, bias, cuts, page=page, decode_tail=tail).double()
            on = torch.sigmoid(torch.tensor(64.0 - 30.0, dtype=torch.float64))
            tol = 1e-5 if dtype == torch.float32 else 1e-2
            assert abs(float(got[698, 0, 0]) - float(on) * 1.0) < tol, (cuts, page)
            assert abs(float(got[63, 1, 1]) - float(on) * 2.0) < tol and abs(float(got[63, 1, 2])) < 1e-6, (cuts, page)
            assert abs(float(got[64, 0, 2]) - float(on) * 3.0) < tol and abs(float(got[64, 0, 3])) < 1e-6, (cuts, page)
            assert abs(float(got[699, 1, 4]) - float(on) * 5.0) < 2 * tol and abs(float(got[699, 1, 0]) - float(on)) < tol, (cuts, page)
            assert float(got[:2].abs().max()) < 1e-6, "the first tokens see nothing that fires"


def check_router(ops, device, E=12, n_groups=4, keep=2, top=3, scale=1.25, T=64):
    g = torch.Generator().manual_seed(4)
    D = 16
    h = torch.randn(T, D, generator=g).double()
    w = {"r.router": torch.randn(E, D, generator=g).double(), "r.correction": (torch.randn(E, generator=g) - 1.0).double()}
    r = dict(experts=E, top=top, scale=scale, groups=dict(count=n_groups, keep=keep))
    chosen, weights = ref.route(h, w, "r.", r)
    logits = (h @ w["r.router"].T).float().to(device)
    ids, wt = ops.moe_route_grouped(logits, w["r.correction"].float().to(device), top, n_groups, keep, scale)
    assert ids.dtype == torch.int32 and wt.dtype == torch.float32
    ids, wt = ids.cpu(), wt.cpu()
    for t in range(T):
        # a close call between two selection scores may go either way in fp32: compare as sets unless the margin is clear
        assert sorted(ids[t].tolist()) == sorted(chosen[t]), f"token {t}: {ids[t].tolist()} for {chosen[t]}"
        for e, c in zip(chosen[t], weights[t]):
            j = ids[t].tolist().index(e)
            assert abs(float(wt[t, j]) - c) < 1e-5
        assert abs(float(wt[t].sum()) - scale) < 1e-5


def check_router_logits(ops, device, T, D=200, E=12):
    g = torch.Generator().manual_seed(9)
    x, w = torch.randn(T, D, generator=g), torch.randn(E, D, generator=g)
    _close(ops.moe_router_logits(x.to(device), w.to(device)), x.double() @ w.double().T, 2e-6, "router logits in fp32")


def check_experts(ops, device, dtype, T=37, D=48, ff=40, E=5, top=2, wide_ok=False, tiled_ok=False, block=None):
    g = torch.Generator().manual_seed(6)
    h = _bf(torch.randn(T, D, generator=g))
    up = _bf(torch.randn(E, ff, D, generator=g) * D ** -0.5)
    down = _bf(torch.randn(E, D, ff, generator=g) * ff ** -0.5)
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    if E > top:                                                     # an idle expert: its pairs go to the one before it
        ids[ids == E - 1] = -1
        for t in range(T):
            if -1 in ids[t].tolist():
                ids[t][ids[t] == -1] = [e for e in range(E - 1) if e not in ids[t].tolist()][0]
    plan = ops.moe_align(ids.to(device), E, wide_ok=wide_ok, tiled_ok=tiled_ok)
    assert block is None or plan.block == block
    a = ops.moe_grouped_linear(h.to(dtype).to(device), up.to(dtype).to(device), plan, gather=True, gelu=True)
    y = ops.moe_grouped_linear(a, down.to(dtype).to(device), plan, gather=False, gelu=False)
    rows = plan.rows.cpu().long()
    assert rows.shape == (T, top) and len(set(rows.reshape(-1).tolist())) == T * top, "every pair has a row of its own"
    want = torch.stack([torch.stack([ref.gelu_erf(h[t] @ up[int(e)].T) @ down[int(e)].T for e in ids[t]]) for t in range(T)])
    _close(y.cpu()[rows], want, 2e-5 if dtype == torch.float32 else 3e-2, "experts over sorted blocks")


def check_side(ops, device, dtype, T=11, D=48, dim=6, L=3, layer=1, V=29, eps=1e-5):
    g = torch.Generator().manual_seed(7)
    x = torch.randn(T, D, generator=g)
    toks = torch.randint(0, V, (T,), generator=g)
    w = {"side.embed": _bf(torch.randn(V, L * dim, generator=g)), f"l{layer}.side.gate": _bf(torch.randn(dim, D, generator=g) * D ** -0.5),
         f"l{layer}.side.proj": _bf(torch.randn(D, dim, generator=g)), f"l{layer}.side.norm": _bf(torch.randn(D, generator=g))}
    want = ref.token_side(x.double(), toks.tolist(), w, layer, dim, eps)
    gate = (x.double() @ w[f"l{layer}.side.gate"].T)
    gm = ops.gelu_tanh_mul_rows(gate.to(dtype).to(device), w["side.embed"].to(dtype).to(device), toks.to(device), layer * dim)
    _close(gm, ref.gelu_tanh(_bf(gate) if dtype != torch.float32 else gate) * w["side.embed"][toks][:, layer * dim:(layer + 1) * dim],
           _tol(dtype), "gelu_tanh(gate) * table slice")
    y = (ref.gelu_tanh(gate) * w["side.embed"][toks][:, layer * dim:(layer + 1) * dim]) @ w[f"l{layer}.side.proj"].T
    xd = x.clone().to(device)
    ops.rmsnorm_residual_add(xd, y.to(dtype).to(device), w[f"l{layer}.side.norm"].to(dtype).to(device), eps)
    _close(xd, want, 2e-5 if dtype == torch.float32 else 2e-2, "the side input")


def check_head_norm_gate(ops, device, dtype, T=6, H=3, dv=20, eps=1e-5):
    g = torch.Generator().manual_seed(8)
    o = torch.randn(T, H, dv, generator=g) * 5
    gate = _bf(torch.randn(T, H * dv + 7, generator=g))
    w = _bf(1 + 0.1 * torch.randn(dv, generator=g))
    for weight in (w, None):
        want = ref.unit_rms(o.double(), eps) * (weight if weight is not None else 1.0)
        want = want.reshape(T, H * dv) * ref.silu(gate[:, 3: 3 + H * dv])
        got = ops.head_rmsnorm_gate(o.to(device), weight.to(dtype).to(device) if weight is not None else None,
                                    gate.to(dtype).to(device)[:, 3: 3 + H * dv], eps, dtype)
        _close(got, want, _tol(dtype), "head norm and gate")
