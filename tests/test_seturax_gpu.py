"""Seturax on the GPU: every HIP kernel of the family against the plain functions of oracle/seturax_ref.py, then the
whole engine (ModelRunner, pools, TraceReplayer, Scheduler) in fp32 and bf16 against the whole-sequence oracle.  Where
random numbers would hide a fault -- one far key among hundreds, the two keys on either side of a window's edge, the
sink -- the inputs are built so that it shows."""
import math

import pytest
import torch

import seturax_util as su
from oracle import seturax_ref as ref

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(autouse=True)
def _product_ops():
    from sglang_custom_amd import ops_backend
    from sglang_custom_amd.distributed import parallel_state

    ops_backend.set_ops_backend(None)      # the HIP library (get_ops() loads it and raises if it is missing)
    parallel_state.init_distributed_environment(1, 0)
    yield


def ops():
    from sglang_custom_amd.ops_backend import get_ops

    return get_ops()


DT = [(torch.float32, 2e-6), (torch.bfloat16, 1e-2)]


# ---------------------------------------------------------------------------------------------- kernels, one by one
@pytest.mark.parametrize("dtype,tol", DT)
@pytest.mark.parametrize("D", [48, 250, 1024])
def test_layernorm_and_token_shift(dtype, tol, D):
    """Two segments of a mixed step (3 tokens continuing a sequence at position 5, 1 token at position 0) and one decode
    token: the first reads the state row, the second zeros, inner tokens their neighbour."""
    g = torch.Generator().manual_seed(D)
    x = torch.randn(5, D, generator=g) * 3 + 1
    w = (1 + 0.1 * torch.randn(D, generator=g)).to(dtype)
    mu = torch.rand(D, generator=g).to(dtype)
    state = torch.randn(4, D, generator=g)
    positions = torch.tensor([5, 6, 7, 0, 9])
    seg_start, seg_len = torch.tensor([0, 3, 4], dtype=torch.int32), torch.tensor([3, 1, 1], dtype=torch.int32)
    tok_req = torch.tensor([0, 0, 0, 1, 2], dtype=torch.int32)
    req_pool = torch.tensor([2, 0, 1])
    req_to_state = torch.tensor([3, 1, 2], dtype=torch.int32)        # request rows 2, 0, 1 -> slots 2, 3, 1
    h_last = torch.zeros(3, D)
    h, hs = ops().layernorm_shift(x.to(DEV), w.to(DEV), 1e-5, shift=mu.to(DEV), state=state.to(DEV), req_to_state=req_to_state.to(DEV),
                                  req_pool_indices=req_pool.to(DEV), positions=positions.to(DEV), h_last=(hl := h_last.to(DEV)),
                                  tok_req=tok_req.to(DEV), seg_start=seg_start.to(DEV), seg_len=seg_len.to(DEV))
    hr = ref.layer_norm(x.double(), w.double(), 1e-5)
    prev = torch.stack([state[2].double(), hr[0], hr[1], torch.zeros(D, dtype=torch.float64), state[1].double()])
    hsr = hr + (prev - hr) * mu.double()
    assert (h.cpu().double() - hr).abs().max() < tol * 8 and (hs.cpu().double() - hsr).abs().max() < tol * 8
    assert (hl.cpu().double() - hr[[2, 3, 4]]).abs().max() < 2e-6 * 8      # the state is fp32 in every dtype
    # decode form: no segment arrays, every token alone
    h2, hs2 = ops().layernorm_shift(x.to(DEV), w.to(DEV), 1e-5, shift=mu.to(DEV), state=state.to(DEV),
                                    req_to_state=torch.arange(5, dtype=torch.int32, device=DEV) % 4,
                                    req_pool_indices=torch.arange(5, device=DEV), positions=positions.to(DEV))
    prev = torch.stack([state[0], state[1], state[2], torch.zeros(D), state[0]]).double()
    assert (hs2.cpu().double() - (hr + (prev - hr) * mu.double())).abs().max() < tol * 8
    assert torch.equal(h2, h)
    assert torch.equal(ops().layernorm_shift(x.to(DEV), w.to(DEV), 1e-5), h)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_bigram_embedding_and_state_commit(dtype):
    V, D, buckets, mp, mc, scale = 50, 40, 7, 37, 13, 4.0
    g = torch.Generator().manual_seed(1)
    table, bigram = torch.randn(V, D, generator=g).to(dtype), torch.randn(buckets + 1, D, generator=g).to(dtype)
    seq = torch.randint(0, V, (9,), generator=g).tolist()
    full = ref.embed(seq, table.double(), bigram.double(), scale, mp, mc, buckets)
    prev_token = torch.zeros(4, dtype=torch.int32, device=DEV)
    rows = torch.zeros(2, 4, D, device=DEV)
    req_to_state = torch.tensor([2, 3], dtype=torch.int32, device=DEV)
    req_pool = torch.tensor([1], device=DEV)            # request row 1 -> slot 3
    got = []
    for lo, hi in ((0, 4), (4, 5), (5, 9)):             # a portion, a single token as a portion, a portion
        ids = torch.tensor(seq[lo:hi], device=DEV)
        seg = dict(tok_req=torch.zeros(hi - lo, dtype=torch.int32, device=DEV), seg_start=torch.zeros(1, dtype=torch.int32, device=DEV),
                   seg_len=torch.tensor([hi - lo], dtype=torch.int32, device=DEV))
        got.append(ops().bigram_embedding(ids, table.to(DEV), bigram.to(DEV), prev_token, req_to_state, req_pool,
                                          torch.arange(lo, hi, device=DEV), scale, mp, mc, buckets, **seg))
        h_last = torch.full((2, 1, D), float(hi), device=DEV)
        ops().commit_sequence_state(rows, prev_token, h_last, ids, req_to_state, req_pool, seg["seg_start"], seg["seg_len"])
        assert int(prev_token[3]) == seq[hi - 1] and float(rows[1, 3, 0]) == hi and float(rows[:, :3].abs().max()) == 0
    assert (torch.cat(got).cpu().double() - full).abs().max() < 1e-5


@pytest.mark.parametrize("dtype,tol", DT)
def test_gelu_mul_and_gated_residual(dtype, tol):
    g = torch.Generator().manual_seed(2)
    T, ff, D = 7, 50, 36
    hp = (torch.randn(T, 2 * ff + 2 * D, generator=g) * 2).to(dtype)
    act = ops().gelu_tanh_and_mul(hp.to(DEV)[:, :ff], hp.to(DEV)[:, ff: 2 * ff])
    want = ref.gelu_tanh(hp[:, :ff].double()) * hp[:, ff: 2 * ff].double()
    assert (act.cpu().double() - want).abs().max() < tol * 16
    x = torch.randn(T, D, generator=g)
    b1, b2 = torch.randn(D, generator=g).to(dtype), torch.randn(D, generator=g).to(dtype)
    y1, y2 = torch.randn(T, D, generator=g).to(dtype), torch.randn(T, D, generator=g).to(dtype)
    g1, g2 = hp[:, 2 * ff: 2 * ff + D], hp[:, 2 * ff + D:]
    want = x.double() + torch.sigmoid(g1.double() + b1.double()) * y1.double() + torch.sigmoid(g2.double() + b2.double()) * y2.double()
    xd, hd = x.to(DEV), hp.to(DEV)
    ops().gated_residual_add(xd, hd[:, 2 * ff: 2 * ff + D], b1.to(DEV), y1.to(DEV), hd[:, 2 * ff + D:], b2.to(DEV), y2.to(DEV))
    assert (xd.cpu().double() - want).abs().max() < 2e-6      # the sum itself is fp32
    xd = x.to(DEV)
    ops().gated_residual_add(xd, hd[:, 2 * ff: 2 * ff + D], b1.to(DEV), y1.to(DEV))
    assert (xd.cpu().double() - (x.double() + torch.sigmoid(g1.double() + b1.double()) * y1.double())).abs().max() < 2e-6


def _latent_case(dtype, H, rank, dr, rot_dims, n_ctx, window, seed, base=10000.0):
    """One sequence of n_ctx cached tokens in scattered slots; returns the pieces both sides need."""
    g = torch.Generator().manual_seed(seed)
    c = torch.randn(n_ctx, rank, generator=g).to(dtype)
    kr = torch.randn(n_ctx, dr, generator=g).to(dtype)          # unrotated rope keys
    slots = torch.randperm(n_ctx + 20, generator=g)[:n_ctx] + 1
    sink = torch.randn(H, generator=g)
    return g, c, kr, slots, sink


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("H,rank,dr,rot_dims,window", [(6, 24, 8, 8, 7), (1, 16, 2, 2, 1), (3, 10, 4, 2, 1000), (40, 8, 4, 4, 33),
                                                      (5, 160, 32, 32, 64), (2, 512, 64, 64, 100)])
def test_latent_norms_rope_write_and_attention(dtype, tol, H, rank, dr, rot_dims, window):
    """The write kernel fills the cache from the projection rows, then attention runs over it three ways that must
    agree with the oracle and with each other: the whole sequence as one portion, portions of unequal size cut by the
    block list, and the last tokens one by one in the decode form."""
    from sglang_custom_amd.layers.rotary_embedding import rotate_half_inv_freq

    n, q_rank, base, eps = 45, 12, 500.0, 1e-5
    g = torch.Generator().manual_seed(H * 1000 + rank)
    a = (torch.randn(n, q_rank + rank + dr + H, generator=g) * 1.5).to(dtype)
    wq, wkv = (1 + 0.1 * torch.randn(q_rank, generator=g)).to(dtype), (1 + 0.1 * torch.randn(rank, generator=g)).to(dtype)
    slots = torch.randperm(n + 19, generator=g)[:n] + 1
    inv_freq = rotate_half_inv_freq(base, rot_dims).to(DEV)
    cache = torch.zeros(n + 20, rank + dr, dtype=dtype, device=DEV)
    pos = torch.arange(n)
    cq = ops().latent_norms_rope_write(a.to(DEV), wq.to(DEV), wkv.to(DEV), pos.to(DEV), slots.to(DEV), inv_freq, cache, q_rank, rank,
                                       dr, rot_dims, eps)
    ad = a.double()
    cq_ref = ref.rms_norm(ad[:, :q_rank], wq.double(), eps)
    c_ref = ref.rms_norm(ad[:, q_rank: q_rank + rank], wkv.double(), eps)
    kr_ref = ref.rotate_half(ad[:, None, q_rank + rank: q_rank + rank + dr], pos, base, rot_dims)[:, 0]
    rows = cache[slots.to(DEV)].cpu().double()
    assert (cq.cpu().double() - cq_ref).abs().max() < tol * 8
    assert (rows - torch.cat([c_ref, kr_ref], 1)).abs().max() < tol * 8
    # attention over the rows the kernel wrote (so that both sides read the same rounded cache)
    qa = torch.randn(n, H, rank, generator=g).to(dtype)
    qr = torch.randn(n, H, dr, generator=g).to(dtype)
    sink = torch.randn(H, generator=g)
    gate = a[:, q_rank + rank + dr:]
    scale = 0.3 / math.sqrt(rank)
    want = ref.absorbed_window_attention(qa.double(), qr.double(), rows[:, :rank], rows[:, rank:], sink.double(), scale, window, base,
                                         rot_dims, gate=gate.double())
    req_to_token = torch.zeros(3, n + 5, dtype=torch.int32)
    req_to_token[1, :n] = slots.to(torch.int32)
    common = dict(req_to_token=req_to_token.to(DEV), sink=sink.to(DEV), inv_freq=inv_freq, rot_dims=rot_dims, window=window, scale=scale)
    bq = ops().latent_window_attention_block_tokens(H, rank, dr, dtype)
    assert bq >= 1

    def blocks_of(portions):
        out, t0 = [], 0
        for m in portions:
            out += [[t0 + k, min(bq, m - k)] for k in range(0, m, bq)]
            t0 += m
        return torch.tensor(out, dtype=torch.int32, device=DEV)

    def run(lo, portions, as_decode=False, num_splits=1):
        """Tokens lo .. of the sequence as one extend batch whose requests are the given portions of it (each request
        the same sequence, with its own prefix), or as a decode batch."""
        m = sum(portions)
        out = torch.zeros(H, m, rank, dtype=dtype, device=DEV)     # head-major memory behind a [T, H, rank] view
        idx = slice(lo, lo + m)
        tok_req = None if as_decode else torch.repeat_interleave(torch.arange(len(portions), dtype=torch.int32),
                                                                 torch.tensor(portions)).to(DEV)
        ops().latent_window_attention(
            qa[idx].to(DEV), qr[idx].to(DEV), cache, out.transpose(0, 1), req_pool_indices=torch.ones(m if as_decode else len(portions), dtype=torch.int64, device=DEV),
            positions=pos[idx].to(DEV), gate=gate[idx].to(DEV), tok_req=tok_req, blocks=None if as_decode else blocks_of(portions),
            num_splits=num_splits, **common)
        return out.transpose(0, 1).cpu().double()

    lim = tol * 4 * max(1.0, float(want.abs().max()))
    assert (run(0, [n]) - want).abs().max() < lim
    assert (run(0, [2, 11, 1, 17, n - 31]) - want).abs().max() < lim
    assert (run(n - 9, [1] * 9, as_decode=True) - want[n - 9:]).abs().max() < lim
    if dtype != torch.float32 and rank <= 512:
        # the keys of every token cut into ranges (some of them empty, one holding the sink) and merged
        for splits in (2, 3, 7):
            assert (run(n - 9, [1] * 9, as_decode=True, num_splits=splits) - want[n - 9:]).abs().max() < lim


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_window_edges_far_keys_and_the_sink_show(dtype):
    """One query at position p = 299 over 300 cached rows with window 128.  All keys score 0 except one planted key whose
    score is large: planted just inside the window (p - 127) the output is that row; just outside (p - 128) it must not
    appear at all; planted far back inside a window of 300, among hundreds, it is found.  With no planted key and a large
    sink, the output shrinks by the sink's share."""
    from sglang_custom_amd.layers.rotary_embedding import rotate_half_inv_freq

    H, rank, dr, n, p = 2, 16, 4, 300, 299
    g = torch.Generator().manual_seed(4)
    values = torch.randn(n, rank, generator=g).to(dtype)
    inv_freq = rotate_half_inv_freq(10000.0, dr).to(DEV)
    req_to_token = (torch.arange(n, dtype=torch.int32) * 2 + 1)[None].to(DEV)      # every other slot

    def attend(planted, window, sink_value, plant_in_rope=False):
        cache = torch.zeros(2 * n + 2, rank + dr, dtype=dtype, device=DEV)
        rows = torch.cat([values, torch.zeros(n, dr, dtype=dtype)], 1)
        qa = torch.zeros(1, H, rank, dtype=dtype)
        qr = torch.zeros(1, H, dr, dtype=dtype)
        if planted is not None and not plant_in_rope:
            # the query looks along the planted row's own direction, and only that row is long in it
            rows[:, 0] = 0
            rows[planted, 0] = 8.0
            qa[:, :, 0] = 8.0
        if planted is not None and plant_in_rope:
            # the same through the rope part: the cache holds rotated keys and the kernel rotates the query by its own
            # position p, so the planted row is the query's direction turned by p
            k = torch.zeros(1, 1, dr, dtype=torch.float64)
            k[..., 0] = 8.0
            rows[planted, rank:] = ref.rotate_half(k, torch.tensor([p]), 10000.0, dr)[0, 0].to(dtype)
            qr[..., 0] = 8.0
        cache[req_to_token[0].long()] = rows.to(DEV)
        sink = torch.full((H,), sink_value, device=DEV)
        out = torch.zeros(1, H, rank, dtype=dtype, device=DEV)
        ops().latent_window_attention(qa.to(DEV), qr.to(DEV), cache, out, req_to_token, torch.zeros(1, dtype=torch.int64, device=DEV),
                                      torch.tensor([p], device=DEV), sink, inv_freq, dr, window, 1.0)
        # the same query as the last token of a prompt portion (the three before it ask for nothing in particular): the
        # run's key range starts earlier than this query's window, so the per-row mask has to cut it
        n_q = min(4, ops().latent_window_attention_block_tokens(H, rank, dr, dtype))
        if n_q > 1:
            qa4 = torch.cat([torch.zeros(n_q - 1, H, rank, dtype=dtype), qa]).to(DEV)
            qr4 = torch.cat([torch.zeros(n_q - 1, H, dr, dtype=dtype), qr]).to(DEV)
            out4 = torch.zeros(n_q, H, rank, dtype=dtype, device=DEV)
            ops().latent_window_attention(qa4, qr4, cache, out4, req_to_token, torch.zeros(1, dtype=torch.int64, device=DEV),
                                          torch.arange(p - n_q + 1, p + 1, device=DEV), sink, inv_freq, dr, window, 1.0,
                                          tok_req=torch.zeros(n_q, dtype=torch.int32, device=DEV),
                                          blocks=torch.tensor([[0, n_q]], dtype=torch.int32, device=DEV))
            assert (out4[-1].float() - out[0].float()).abs().max() < (1e-5 if dtype == torch.float32 else 1e-2), \
                "a query answers differently inside a prompt portion"
        return out[0, 0].cpu().double(), rows.double()

    tol = 1e-4 if dtype == torch.float32 else 2e-2
    for rope in (False, True):
        o, rows = attend(p - 127, 128, -30.0, rope)
        assert (o - rows[p - 127, :rank]).abs().max() < tol, "the oldest key inside the window"
        o, rows = attend(p - 128, 128, -30.0, rope)
        mean_in = rows[p - 127: p + 1, :rank].mean(0)
        assert (o - mean_in).abs().max() < tol, "a key just outside the window leaked in"
        o, rows = attend(3, 300, -30.0, rope)
        assert (o - rows[3, :rank]).abs().max() < tol, "a far key among hundreds"
        o, rows = attend(0, 300, -30.0, rope)
        assert (o - rows[0, :rank]).abs().max() < tol, "the first token of the sequence"
    o, rows = attend(None, 128, math.log(128.0))         # 128 keys of weight 1 and a sink of weight 128: half
    assert (o - 0.5 * rows[p - 127: p + 1, :rank].mean(0)).abs().max() < tol
    o, rows = attend(None, 1, -30.0)
    assert (o - rows[p, :rank]).abs().max() < tol, "a window of one sees the token itself"


# ---------------------------------------------------------------------------------------------- the engine
CASES = [("float32", 3e-5), ("bfloat16", 6e-2)]


@pytest.mark.parametrize("dtype,tol", CASES)
def test_prefill_decode_portions_and_batches_against_the_oracle(dtype, tol):
    cfg = su.make_config()
    w = su.make_weights(cfg, seed=3)
    mr = su.build_runner(cfg, w, dtype=dtype, device=DEV, max_total_tokens=192, max_running_requests=3)
    # more than 64 rows at once: the prefill-sized GEMM paths, on widths that are multiples of nothing in particular
    long = su.random_prompts(cfg, [150], seed=4)
    su.replay_and_compare(mr, cfg, w, long, [[("r0", 150)]], tol)
    su.replay_and_compare(mr, cfg, w, long, [[("r0", 71)], [("r0", 2)], [("r0", 77)]], tol)
    p = su.random_prompts(cfg, [23], seed=0)
    su.replay_and_compare(mr, cfg, w, p, [[("r0", 23)]], tol)
    su.replay_and_compare(mr, cfg, w, p, [[("r0", 1)] for _ in range(23)], tol)
    su.replay_and_compare(mr, cfg, w, p, [[("r0", k)] for k in (2, 2, 3, 5, 2, 7, 1, 1)], tol)
    prompts = su.random_prompts(cfg, [17, 9, 1, 12, 20, 6], seed=7)
    sched = [[("r0", 5), ("r1", 2)], [("r0", 1), ("r1", 7), ("r2", 1)], [("r0", 4), ("r3", 3)], [("r3", 1)],
             [("r0", 1), ("r3", 1)], [("r0", 6), ("r3", 7), ("r4", 2)], [("r4", 1), ("r5", 1)], [("r4", 1), ("r5", 1)],
             [("r4", 9), ("r5", 4)], [("r4", 1)], [("r4", 6)]]
    for _ in range(2):        # the second pass runs on used slots, rows and state
        su.replay_and_compare(mr, cfg, w, prompts, sched, tol)
        assert su.pools_are_whole(mr)


@pytest.mark.parametrize("dtype,tol", CASES)
@pytest.mark.parametrize("page_size", [1, 16])
def test_long_decode_across_windows_and_pages(dtype, tol, page_size):
    """Sizes unlike the small default: 5 and 40 heads, a 96-wide latent, windows of 33 and 70 that a 150-token decode
    crosses twice, a layer without feed-forward, pages of 16."""
    layers = [(su.mixer(5, 16, 8, 24, 96, 40, 33), 120), (su.mixer(40, 4, 4, 4, 16, 20, 70, base=300.0), None),
              (su.mixer(2, 32, 16, 16, 64, 24, 33), 72)]
    cfg = su.make_config(width=80, vocab=97, layers=layers, buckets=101, mul_prev=5, mul_cur=9, scale=8.0, logit_scale=0.3)
    w = su.make_weights(cfg, seed=21)
    mr = su.build_runner(cfg, w, dtype=dtype, device=DEV, max_total_tokens=512, max_running_requests=2, page_size=page_size)
    p = su.random_prompts(cfg, [190, 75], seed=3)
    sched = [[("r0", 40), ("r1", 2)]] + [[("r0", 1), ("r1", 1)] for _ in range(73)] + [[("r0", 1)] for _ in range(77)]
    su.replay_and_compare(mr, cfg, w, p, sched, tol)
    su.replay_and_compare(mr, cfg, w, p, [[("r1", 75)], [("r0", 100)], [("r0", 31)], [("r0", 2)], [("r0", 57)]], tol)
    assert su.pools_are_whole(mr)


@pytest.mark.parametrize("dtype,tol", CASES)
def test_equal_and_unit_sizes(dtype, tol):
    """One head, rope width equal to the head width, value width equal to the rank, rank 2, window 1 and a window longer
    than any prompt, width equal to the vocabulary, one bigram bucket."""
    layers = [(su.mixer(1, 4, 4, 8, 8, 8, 1), 8), (su.mixer(4, 2, 2, 2, 2, 2, 1000), None)]
    cfg = su.make_config(width=16, vocab=16, layers=layers, buckets=1, mul_prev=1, mul_cur=1, scale=1.0, logit_scale=1.0)
    w = su.make_weights(cfg, seed=11)
    prompts = su.random_prompts(cfg, [14, 5], seed=1)
    mr = su.build_runner(cfg, w, dtype=dtype, device=DEV, max_total_tokens=32)
    su.replay_and_compare(mr, cfg, w, prompts, [[("r0", 3), ("r1", 1)], [("r0", 1), ("r1", 1)], [("r0", 10), ("r1", 3)]], tol)
    assert su.pools_are_whole(mr)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_scheduler(dtype):
    """The engine's own entry point, prompts chunked and decode tokens riding prefill batches.  fp32 must give the
    oracle's tokens; bf16 must give the same tokens whether a prompt is chunked or not, up to a near-tie."""
    from sglang_custom_amd.managers.schedule_batch import Req
    from sglang_custom_amd.managers.scheduler import Scheduler
    from sglang_custom_amd.sampling.sampling_params import SamplingParams

    cfg = su.make_config()
    w = su.make_weights(cfg, seed=3)
    prompts = su.random_prompts(cfg, [11, 3, 7, 15, 1], seed=9)
    outs = []
    for chunk, mixed in ((None, False), (6, True)):
        mr = su.build_runner(cfg, w, dtype=dtype, device=DEV, max_total_tokens=96, max_running_requests=3,
                             chunked_prefill_size=chunk, enable_mixed_chunk=mixed)
        sch = Scheduler(mr)
        for k, p in prompts.items():
            sch.add_request(Req(k, p, SamplingParams(temperature=0, max_new_tokens=6)))
        done = sch.run_until_done()
        outs.append({k: done[k].output_ids for k in prompts})
        assert su.pools_are_whole(mr)
    if dtype == "float32":
        for k, p in prompts.items():
            assert outs[0][k] == outs[1][k] == ref.greedy(cfg, w, p, 6), k
    else:
        same = sum(outs[0][k] == outs[1][k] for k in prompts)
        assert same >= len(prompts) - 1


def _write_model_folder(folder, cfg, weights):
    """config.json + model.safetensors (8-byte header length, JSON header, raw little-endian data), written by hand."""
    import json
    import struct

    header, blobs, at = {}, [], 0
    for name, t in weights.items():
        raw = t.contiguous().view(torch.int16).numpy().tobytes() if t.dtype == torch.bfloat16 else t.contiguous().numpy().tobytes()
        kind = {torch.bfloat16: "BF16", torch.float32: "F32", torch.int32: "I32"}[t.dtype]
        header[name] = {"dtype": kind, "shape": list(t.shape), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    head = json.dumps(header).encode()
    head += b" " * (-len(head) % 8)
    with open(folder / "model.safetensors", "wb") as f:
        f.write(struct.pack("<Q", len(head)) + head + b"".join(blobs))
    with open(folder / "config.json", "w") as f:
        json.dump(cfg, f)


@pytest.mark.parametrize("dtype,tol", CASES)
def test_command_line_replay_of_a_model_folder(tmp_path, dtype, tol):
    """bin/trace_run as a user starts it: a model folder on disk, steps on standard input, logits in files; four live
    requests at most, a pool that the requests' total would not fit into."""
    import json
    import os
    import subprocess
    import sys

    import numpy as np

    layers = [(su.mixer(6, 16, 8, 16, 32, 24, 11), 96), (su.mixer(3, 8, 4, 12, 20, 16, 64, base=777.0), None)]
    cfg = su.make_config(width=64, vocab=83, layers=layers, buckets=29, mul_prev=11, mul_cur=5, scale=2.0, logit_scale=0.75)
    w = su.make_weights(cfg, seed=17)
    _write_model_folder(tmp_path, cfg, w)
    prompts = su.random_prompts(cfg, [70, 33, 1, 64, 40], seed=6)
    sched = [[("r0", 40), ("r1", 2)], [("r0", 1), ("r1", 30), ("r2", 1), ("r3", 7)], [("r0", 29), ("r1", 1), ("r3", 57)],
             [("r4", 2)], [("r4", 1)], [("r4", 37)]]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    lines, want, at = [], [], {k: 0 for k in prompts}
    full = {k: ref.forward(cfg, w, p) for k, p in prompts.items()}
    for n, step in enumerate(sched):
        entries, rows, end = [], [], []
        for name, cnt in step:
            lo, hi = at[name], at[name] + cnt
            asked = list(range(0, cnt, 3)) + ([cnt - 1] if (cnt - 1) % 3 else [])
            entries.append({"id": name, "tokens": prompts[name][lo:hi], "want": asked})
            rows.append(full[name][lo:hi][asked])
            at[name] = hi
            if hi == len(prompts[name]):
                end.append(name)
        lines.append(json.dumps({"step": n, "entries": entries, "end": end}))
        want.append(torch.cat(rows))
    lines.append(json.dumps({"step": len(sched), "entries": [], "end": []}))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(tmp_path), "--dtype", dtype, "--out", str(out),
                        "--max-tokens", "192"], input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=300, cwd=root)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [x for x in r.stdout.split("\n") if x.startswith("done")] == [f"done {n}" for n in range(len(sched) + 1)]
    for n, expect in enumerate(want):
        got = torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(-1, cfg["vocab"]).copy())
        assert got.shape == expect.shape
        assert su.rel_err(got, expect) < tol, f"step {n}"
    assert not (out / f"{len(sched)}.f32").exists()
