"""Verozen on the CPU: the package's host side (configuration, weight stacking, model wiring, ScheduleBatch /
ForwardBatch, the KV / request / state pools, TraceReplayer, Scheduler) runs with the CPU stand-in ops (tests/cpu_ops.py)
and every logit is compared with the plain whole-sequence implementation in oracle/verozen_ref.py.  The HIP kernels
have their own file (test_verozen_gpu.py); here the arithmetic is the stand-in's, the bookkeeping is the package's."""
import pytest
import torch

import verozen_cases as cases
import verozen_util as vu
from oracle import verozen_ref as ref

TOL = 2e-5


@pytest.fixture(autouse=True)
def _cpu_backend():
    import cpu_ops
    from sglang_custom_amd import ops_backend
    from sglang_custom_amd.distributed import parallel_state

    prev = ops_backend._backend
    ops_backend.set_ops_backend(cpu_ops)
    parallel_state.init_distributed_environment(1, 0)
    yield
    ops_backend.set_ops_backend(prev)


@pytest.fixture(scope="module")
def model():
    cfg = vu.make_config()
    return cfg, vu.make_weights(cfg, seed=3)


def test_oracle_recurrences_agree_with_their_step_form():
    """The oracle states both recurrences as explicit sums over earlier tokens; stepping the matrix gives the same."""
    g = torch.Generator().manual_seed(0)
    T, H, d, dv = 13, 2, 5, 4
    q, k, v = (torch.randn(T, H, n, generator=g, dtype=torch.float64) for n in (d, d, dv))
    log_a = -torch.rand(T, H, d, generator=g, dtype=torch.float64)
    S = torch.zeros(H, d, dv, dtype=torch.float64)
    S2 = torch.zeros(H, d, dv, dtype=torch.float64)
    decay = [0.9, 0.6]
    for t in range(T):
        S = torch.exp(log_a[t])[:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        S2 = torch.tensor(decay, dtype=torch.float64)[:, None, None] * S2 + k[t][:, :, None] * v[t][:, None, :]
        assert (torch.einsum("hkv,hk->hv", S, q[t]) - ref.decayed_sum_per_channel(q, k, v, log_a)[t]).abs().max() < 1e-10
        assert (torch.einsum("hkv,hk->hv", S2, q[t]) - ref.decayed_sum_per_head(q, k, v, decay)[t]).abs().max() < 1e-10


@pytest.mark.parametrize("kind", ["gla", "attention", "retention"])
def test_each_mixer_alone(kind):
    """One-layer models of a single mixer each, without feed-forward and side input: whole, cut, and token by token."""
    mixer = dict(gla=vu.gla(), attention=vu.attention(), retention=vu.retention())[kind]
    cfg = vu.make_config(layers=[(mixer, None)], side=0)
    w = vu.make_weights(cfg, seed=1)
    prompts = vu.random_prompts(cfg, [19])
    mr = vu.build_runner(cfg, w)
    vu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 19)]], TOL)
    vu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 7)], [("r0", 2)]] + [[("r0", 1)] for _ in range(10)], TOL)
    assert vu.pools_are_whole(mr)


def test_whole_prompt_then_token_by_token(model):
    cfg, w = model
    prompts = vu.random_prompts(cfg, [23])
    mr = vu.build_runner(cfg, w)
    vu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 23)]], TOL)
    vu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 1)] for _ in range(23)], TOL)
    vu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 9)]] + [[("r0", 1)] for _ in range(14)], TOL)
    assert vu.pools_are_whole(mr)


@pytest.mark.parametrize("sizes", [[2, 2, 2, 3, 5, 2, 7, 1, 1, 2], [1, 4, 4, 4, 4, 4, 4, 2], [25, 2]])
def test_portions_of_any_size(model, sizes):
    cfg, w = model
    prompts = vu.random_prompts(cfg, [sum(sizes)], seed=5)
    mr = vu.build_runner(cfg, w)
    vu.replay_and_compare(mr, cfg, w, prompts, [[("r0", k)] for k in sizes], TOL)
    assert vu.pools_are_whole(mr)


@pytest.mark.parametrize("page_size", [1, 4])
def test_mixed_batches_reuse_slots_and_pages(model, page_size):
    """Unequal requests side by side -- portions beside single tokens, a request that sits a step out, requests that end
    while others go on -- in a pool so small that KV slots, request rows and state slots are all handed out again."""
    cfg, w = model
    prompts = vu.random_prompts(cfg, [17, 9, 1, 12, 20, 6], seed=7)
    sched = [[("r0", 5), ("r1", 2)], [("r0", 1), ("r1", 7), ("r2", 1)], [("r0", 4), ("r3", 3)], [("r3", 1)],
             [("r0", 1), ("r3", 1)], [("r0", 6), ("r3", 7), ("r4", 2)], [("r4", 1), ("r5", 1)], [("r4", 1), ("r5", 1)],
             [("r4", 9), ("r5", 4)], [("r4", 1)], [("r4", 6)]]
    mr = vu.build_runner(cfg, w, max_total_tokens=48, max_running_requests=3, page_size=page_size)
    vu.replay_and_compare(mr, cfg, w, prompts, sched, TOL)
    assert vu.pools_are_whole(mr)
    # the same again on the used pools: stale keys, stale matrices
    vu.replay_and_compare(mr, cfg, w, prompts, sched, TOL)
    assert vu.pools_are_whole(mr)


def test_equal_and_unit_sizes():
    """Sizes that a model may happen to make equal or 1: one norm group, one head, as many key heads as query heads, no
    rotation and a rotation of the whole head, one expert group, every group kept, one expert per token, a residual weight
    of 1, a layer without feed-forward that still has its second norm, no side input, width equal to the vocabulary."""
    layers = [(vu.attention(heads=2, kv_heads=2, dim=8, rot_dims=8), vu.moe(experts=3, top=1, count=1, keep=1, ff=8)),
              (vu.retention(heads=1, dim=4, vdim=4, rot_dims=0, decay=(1.0,)), None),
              (vu.gla(heads=1, dim=8, vdim=8, tau=1.0, rank=1), vu.moe(experts=4, top=4, count=4, keep=4, ff=4, scale=1.0)),
              (vu.attention(heads=3, kv_heads=1, dim=4, rot_dims=0), None)]
    cfg = vu.make_config(layers=layers, width=16, vocab=16, groups=1, alpha=1.0, side=0)
    w = vu.make_weights(cfg, seed=11, norm2_without_mlp=True)
    prompts = vu.random_prompts(cfg, [14, 5], seed=1)
    mr = vu.build_runner(cfg, w, max_total_tokens=32)
    vu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 3), ("r1", 1)], [("r0", 1), ("r1", 1)], [("r0", 10), ("r1", 3)]], TOL)


def test_state_is_what_the_next_step_reads(model):
    """Cutting a prompt must hand over exactly the layers' matrices: a corrupted matrix changes the next portion's logits,
    a sequence's first token reads none of what its slot held, and a finished request's slot goes to the next one."""
    cfg, w = model
    from sglang_custom_amd.managers.trace_replay import TraceReplayer

    prompts = vu.random_prompts(cfg, [8], seed=2)["r0"]
    mr = vu.build_runner(cfg, w)
    pool = mr.req_to_token_pool.state_pool
    assert sorted(pool.matrices) == [0, 2, 3] and pool.matrices[2].shape[1:] == (2, 12, 20)
    for m in pool.matrices.values():
        m.fill_(123.0)
    rp = TraceReplayer(mr)
    want = ref.forward(vu.public(cfg), w, prompts)
    assert vu.rel_err(rp.step([dict(id="a", tokens=prompts[:4], want=[0, 1, 2, 3])]), want[:4]) < TOL
    slot = rp.live["a"].state_slot
    good = {l: m[slot].clone() for l, m in pool.matrices.items()}
    pool.matrices[2][slot] += 0.5
    assert vu.rel_err(rp.step([dict(id="a", tokens=prompts[4:5], want=[0])]), want[4:5]) > 1e-3
    rp.finish("a")
    rp.step([dict(id="b", tokens=prompts[:4], want=[])])
    assert rp.live["b"].state_slot is not None
    for l, m in pool.matrices.items():
        assert torch.equal(m[rp.live["b"].state_slot], good[l])
    assert vu.rel_err(rp.step([dict(id="b", tokens=prompts[4:], want=[0, 1, 2, 3])], ["b"]), want[4:]) < TOL
    assert vu.pools_are_whole(mr)


@pytest.mark.parametrize("chunk,mixed", [(None, False), (6, False), (6, True)])
def test_greedy_generation_through_the_scheduler(model, chunk, mixed):
    """The package's own entry point: requests queued at the Scheduler, prompts chunked by its policy, decode batches
    (and decode tokens riding prefill batches) formed by it, tokens picked by the Sampler."""
    from sglang_custom_amd.managers.schedule_batch import Req
    from sglang_custom_amd.managers.scheduler import Scheduler
    from sglang_custom_amd.sampling.sampling_params import SamplingParams

    cfg, w = model
    prompts = vu.random_prompts(cfg, [11, 3, 7, 15, 1], seed=9)
    mr = vu.build_runner(cfg, w, max_total_tokens=96, max_running_requests=3, chunked_prefill_size=chunk, enable_mixed_chunk=mixed)
    sch = Scheduler(mr)
    for k, p in prompts.items():
        sch.add_request(Req(k, p, SamplingParams(temperature=0, max_new_tokens=6)))
    done = sch.run_until_done()
    for k, p in prompts.items():
        assert done[k].output_ids == ref.greedy(vu.public(cfg), w, p, 6), k
    assert vu.pools_are_whole(mr)
    if chunk:
        assert sch.num_prefill_batches > 3


def test_prefix_cache_is_refused(model):
    from sglang_custom_amd.managers.scheduler import Scheduler

    cfg, w = model
    with pytest.raises(ValueError):
        Scheduler(vu.build_runner(cfg, w), enable_radix_cache=True)


def test_configuration_is_read_not_assumed():
    from sglang_custom_amd.configs.model_config import ModelConfig
    from sglang_custom_amd.models.registry import get_model_class

    cfg = vu.public(vu.make_config())
    mc = ModelConfig(cfg, dtype="float32")
    assert mc.architecture == "Verozen" and get_model_class(mc.architecture).__name__ == "VerozenForCausalLM"
    assert mc.kv_layer_shapes == [None, (2, 16, 16), None, None]
    assert mc.recurrent_layer_shapes == [(3, 8, 12), None, (2, 12, 20), (1, 20, 4)]
    assert mc.norm_groups == 3 and mc.postln_alpha == 2.0 and mc.token_side_dim == 6
    for key, value in (("type", "something_else"),):
        bad = vu.public(vu.make_config())
        bad["layers"][1][key] = value
        with pytest.raises(ValueError):
            ModelConfig(bad)
    bad = vu.public(vu.make_config())
    bad["layers"][2]["mixer"]["decay"] = [0.5]
    with pytest.raises(ValueError):
        ModelConfig(bad)


# ---- the stand-in ops themselves against the oracle's functions: the same cases the HIP kernels run on the GPU
def test_standins_norms_rotations_gates():
    import cpu_ops

    cases.check_group_norm(cpu_ops, "cpu", torch.float32)
    cases.check_group_norm(cpu_ops, "cpu", torch.float32, D=40, groups=1)
    for inter in (True, False):
        cases.check_head_norm_rope(cpu_ops, "cpu", torch.float32, inter, rot_dims=16)
        cases.check_head_norm_rope(cpu_ops, "cpu", torch.float32, inter, rot_dims=24, with_norm=False, scale=1.0)
    cases.check_head_norm_gate(cpu_ops, "cpu", torch.float32)
    cases.check_side(cpu_ops, "cpu", torch.float32)


def test_standins_recurrence_attention_mixture():
    import cpu_ops

    cases.check_recurrence(cpu_ops, "cpu", torch.float32, per_channel=True, cuts=(20, 2, 1, 22))
    cases.check_recurrence(cpu_ops, "cpu", torch.float32, per_channel=False, cuts=(3, 40, 1, 1), decode_tail=2)
    cases.check_sigmoid_attention(cpu_ops, "cpu", torch.float32, T=40, cuts=(17, 2, 20, 1), decode_tail=1)
    cases.check_router(cpu_ops, "cpu")
    cases.check_router(cpu_ops, "cpu", E=8, n_groups=8, keep=3, top=2)
    cases.check_experts(cpu_ops, "cpu", torch.float32)
    cases.check_router_logits(cpu_ops, "cpu", 5)
