"""Verozen on the GPU: every HIP kernel of the family against the plain functions of oracle/verozen_ref.py
(verozen_cases.py holds the cases), then the whole engine (ModelRunner, pools, TraceReplayer, Scheduler) in fp32 and bf16
against the whole-sequence oracle.  Where random numbers would hide a fault -- one far key among hundreds, the key a
query may just see and the one it may just not, a page's border, the first tokens of a sequence, a stale matrix in a
reused slot -- the inputs are built so that it shows."""
import pytest
import torch

import verozen_cases as cases
import verozen_util as vu
from oracle import verozen_ref as ref

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]


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


# ---------------------------------------------------------------------------------------------- kernels, one by one
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D,groups", [(48, 3), (40, 1), (1024, 4), (96, 32)])
def test_group_norm_and_normed_add(dtype, D, groups):
    cases.check_group_norm(ops(), DEV, dtype, D=D, groups=groups)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("interleaved", [True, False])
@pytest.mark.parametrize("d,rot_dims,with_norm", [(24, 16, True), (24, 24, False), (128, 64, True), (6, 0, True), (200, 2, False)])
def test_head_norm_and_rotation(dtype, interleaved, d, rot_dims, with_norm):
    cases.check_head_norm_rope(ops(), DEV, dtype, interleaved, rot_dims, d=d, with_norm=with_norm)


@pytest.mark.parametrize("dtype", DTYPES)
def test_head_norm_gate_and_side_input(dtype):
    cases.check_head_norm_gate(ops(), DEV, dtype)
    cases.check_head_norm_gate(ops(), DEV, dtype, H=1, dv=128)
    cases.check_side(ops(), DEV, dtype)
    cases.check_side(ops(), DEV, dtype, dim=1, L=1, layer=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("per_channel", [True, False])
@pytest.mark.parametrize("dk,dv,H", [(12, 20, 3), (32, 32, 4), (64, 64, 2), (128, 96, 1), (200, 33, 2), (1, 1, 1)])
def test_recurrence_whole_cut_and_decoded(dtype, per_channel, dk, dv, H):
    for cuts, tail in (((45,), 0), ((20, 2, 1, 22), 0), ((17, 16, 2) + (1,) * 10, 10), ((1,) * 45, 45)):
        cases.check_recurrence(ops(), DEV, dtype, per_channel, H=H, dk=dk, dv=dv, cuts=cuts, decode_tail=tail)


@pytest.mark.parametrize("dtype", DTYPES)
def test_recurrence_far_keys_first_tokens_and_slots(dtype):
    cases.check_recurrence_far_key(ops(), DEV, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,d", [(4, 2, 32), (8, 1, 64), (3, 3, 24), (32, 1, 32), (6, 2, 128), (1, 1, 8), (4, 2, 96), (2, 1, 160),
                                   (128, 1, 32), (2, 2, 256)])
def test_sigmoid_attention_whole_cut_and_decoded(dtype, H, G, d):
    """Multiples of 32 run on the matrix cores in bf16 (96 and 160: tiles whose chunk counts are no power of two, column
    tiles that do not fill the four waves; 256: the widest), 24 and 8 on the vector ALU; 128 heads on one key head is two
    workgroups per run on the matrix cores, eight on the vector ALU."""
    for cuts, tail, page, splits in (((150,), 0, 1, 1), ((63, 2, 1, 84), 0, 64, 1), ((140,) + (1,) * 10, 10, 16, 1),
                                     ((146, 1, 1, 1, 1), 4, 1, 3)):
        cases.check_sigmoid_attention(ops(), DEV, dtype, H=H, G=G, d=d, cuts=cuts, decode_tail=tail, page=page, splits=splits)


@pytest.mark.parametrize("dtype", DTYPES)
def test_sigmoid_attention_far_keys_and_the_causal_edge(dtype):
    cases.check_sigmoid_attention_planted(ops(), DEV, dtype)


def test_router_groups_corrections_and_ties():
    cases.check_router(ops(), DEV)
    cases.check_router(ops(), DEV, E=8, n_groups=8, keep=3, top=2)          # groups of one
    cases.check_router(ops(), DEV, E=6, n_groups=1, keep=1, top=6)          # everything chosen
    cases.check_router(ops(), DEV, E=160, n_groups=8, keep=4, top=8, T=300)
    # equal selection scores: the smaller index wins, and -inf never does while something is left
    logits = torch.zeros(2, 8, device=DEV)
    ids, w = ops().moe_route_grouped(logits, torch.full((8,), -3.0, device=DEV), 3, 4, 2, 2.0)
    assert ids.cpu().tolist() == [[0, 1, 2]] * 2 and torch.allclose(w.cpu(), torch.full((2, 3), 2.0 / 3))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,D,ff,E,top", [(37, 48, 40, 5, 2), (300, 64, 96, 8, 4), (1, 32, 8, 3, 1), (70, 50, 36, 4, 3)])
def test_experts_over_sorted_blocks(dtype, T, D, ff, E, top):
    cases.check_experts(ops(), DEV, dtype, T=T, D=D, ff=ff, E=E, top=top)


@pytest.mark.parametrize("D,ff", [(64, 96), (200, 72), (256, 128)])
def test_experts_over_wide_blocks(D, ff):
    """Enough rows per expert for the 128-row blocks of the prefill-sized kernel: K tiles with a tail (200, 72), one idle
    expert, column counts that are no multiple of the tile."""
    cases.check_experts(ops(), DEV, torch.bfloat16, T=1100, D=D, ff=ff, E=4, top=2, wide_ok=True, block=128)


@pytest.mark.parametrize("D,ff", [(128, 192), (256, 128)])
def test_experts_over_blocks_of_the_prefill_projection_kernel(D, ff):
    """Blocks of 256 rows on the package's prefill GEMM kernel with per-block weights, gathered rows and the activation in
    its epilogue: widths that are multiples of 64, one idle expert, a partly filled last block per expert."""
    cases.check_experts(ops(), DEV, torch.bfloat16, T=2300, D=D, ff=ff, E=4, top=2, tiled_ok=True, block=256)


def test_router_logits_few_rows_and_many():
    for T in (1, 5, 64, 300):
        cases.check_router_logits(ops(), DEV, T)


# ---------------------------------------------------------------------------------------------- the engine
CASES = [("float32", 3e-5), ("bfloat16", 6e-2)]


@pytest.mark.parametrize("dtype,tol", CASES)
@pytest.mark.parametrize("kind", ["gla", "attention", "retention"])
def test_each_mixer_alone(dtype, tol, kind):
    mixer = dict(gla=vu.gla(), attention=vu.attention(), retention=vu.retention())[kind]
    cfg = vu.make_config(layers=[(mixer, None)], side=0)
    w = vu.make_weights(cfg, seed=1)
    prompts = vu.random_prompts(cfg, [90])
    mr = vu.build_runner(cfg, w, dtype=dtype, device=DEV)
    vu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 90)]], tol)
    vu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 66)], [("r0", 2)]] + [[("r0", 1)] for _ in range(22)], tol)
    assert vu.pools_are_whole(mr)


@pytest.mark.parametrize("dtype,tol", CASES)
def test_prefill_decode_portions_and_batches_against_the_oracle(dtype, tol):
    cfg = vu.make_config()
    w = vu.make_weights(cfg, seed=3, separated_router=dtype != "float32")
    mr = vu.build_runner(cfg, w, dtype=dtype, device=DEV, max_total_tokens=192, max_running_requests=3)
    # more than 64 rows at once: the prefill-sized GEMM paths, on widths that are multiples of nothing in particular
    long = vu.random_prompts(cfg, [150], seed=4)
    vu.replay_and_compare(mr, cfg, w, long, [[("r0", 150)]], tol)
    vu.replay_and_compare(mr, cfg, w, long, [[("r0", 71)], [("r0", 2)], [("r0", 77)]], tol)
    p = vu.random_prompts(cfg, [23], seed=0)
    vu.replay_and_compare(mr, cfg, w, p, [[("r0", 23)]], tol)
    vu.replay_and_compare(mr, cfg, w, p, [[("r0", 1)] for _ in range(23)], tol)
    vu.replay_and_compare(mr, cfg, w, p, [[("r0", k)] for k in (2, 2, 3, 5, 2, 7, 1, 1)], tol)
    prompts = vu.random_prompts(cfg, [17, 9, 1, 12, 20, 6], seed=7)
    sched = [[("r0", 5), ("r1", 2)], [("r0", 1), ("r1", 7), ("r2", 1)], [("r0", 4), ("r3", 3)], [("r3", 1)],
             [("r0", 1), ("r3", 1)], [("r0", 6), ("r3", 7), ("r4", 2)], [("r4", 1), ("r5", 1)], [("r4", 1), ("r5", 1)],
             [("r4", 9), ("r5", 4)], [("r4", 1)], [("r4", 6)]]
    for _ in range(2):        # the second pass runs on used slots, rows and matrices
        vu.replay_and_compare(mr, cfg, w, prompts, sched, tol)
        assert vu.pools_are_whole(mr)


@pytest.mark.parametrize("dtype,tol", CASES)
@pytest.mark.parametrize("page_size", [1, 16])
def test_long_decode_on_other_sizes(dtype, tol, page_size):
    """Sizes unlike the small default, on the matrix-core paths in bf16: heads of 64 and 32, 8 query heads on 2 key heads,
    16 experts in 4 groups, a 150-token decode over pages of 16, two requests side by side."""
    layers = [(vu.gla(heads=2, dim=64, vdim=32, tau=8.0, rank=8), vu.moe(experts=16, top=4, count=4, keep=2, ff=64)),
              (vu.attention(heads=8, kv_heads=2, dim=32, rot_dims=16, base=5000.0, scale=0.18), vu.moe(experts=4, top=2, count=2, keep=1, ff=96)),
              (vu.retention(heads=3, dim=32, vdim=64, rot_dims=32, base=300.0, decay=(0.99, 0.9, 1.0)), None),
              (vu.attention(heads=2, kv_heads=2, dim=64, rot_dims=64, base=100.0, scale=0.12), vu.moe(experts=8, top=8, count=1, keep=1, ff=32))]
    cfg = vu.make_config(layers=layers, width=128, vocab=97, groups=8, alpha=1.5, side=8)
    w = vu.make_weights(cfg, seed=21, separated_router=dtype != "float32")
    mr = vu.build_runner(cfg, w, dtype=dtype, device=DEV, max_total_tokens=512, max_running_requests=2, page_size=page_size)
    p = vu.random_prompts(cfg, [190, 75], seed=3)
    sched = [[("r0", 40), ("r1", 2)]] + [[("r0", 1), ("r1", 1)] for _ in range(73)] + [[("r0", 1)] for _ in range(77)]
    vu.replay_and_compare(mr, cfg, w, p, sched, tol)
    vu.replay_and_compare(mr, cfg, w, p, [[("r1", 75)], [("r0", 100)], [("r0", 31)], [("r0", 2)], [("r0", 57)]], tol)
    assert vu.pools_are_whole(mr)


@pytest.mark.parametrize("dtype,tol", CASES)
def test_equal_and_unit_sizes(dtype, tol):
    """The sizes of the CPU test of this name.  The single-head layers keep a width of 8: a head of 4 values divided by its
    root mean square turns bf16 noise into a large change of direction whenever the head's output is near zero."""
    layers = [(vu.attention(heads=2, kv_heads=2, dim=8, rot_dims=8), vu.moe(experts=3, top=1, count=1, keep=1, ff=8)),
              (vu.retention(heads=1, dim=4, vdim=4, rot_dims=0, decay=(1.0,)), None),
              (vu.gla(heads=1, dim=8, vdim=8, tau=1.0, rank=1), vu.moe(experts=4, top=4, count=4, keep=4, ff=4, scale=1.0)),
              (vu.attention(heads=3, kv_heads=1, dim=4, rot_dims=0), None)]
    cfg = vu.make_config(layers=layers, width=16, vocab=16, groups=1, alpha=1.0, side=0)
    w = vu.make_weights(cfg, seed=11, norm2_without_mlp=True, separated_router=dtype != "float32")
    prompts = vu.random_prompts(cfg, [14, 5], seed=1)
    mr = vu.build_runner(cfg, w, dtype=dtype, device=DEV, max_total_tokens=32)
    vu.replay_and_compare(mr, cfg, w, prompts, [[("r0", 3), ("r1", 1)], [("r0", 1), ("r1", 1)], [("r0", 10), ("r1", 3)]], tol)
    assert vu.pools_are_whole(mr)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_scheduler(dtype):
    """The engine's own entry point, prompts chunked and decode tokens riding prefill batches.  fp32 must give the
    oracle's tokens; bf16 must give the same tokens whether a prompt is chunked or not, up to a near-tie."""
    from sglang_custom_amd.managers.schedule_batch import Req
    from sglang_custom_amd.managers.scheduler import Scheduler
    from sglang_custom_amd.sampling.sampling_params import SamplingParams

    cfg = vu.make_config()
    w = vu.make_weights(cfg, seed=3)
    prompts = vu.random_prompts(cfg, [11, 3, 7, 15, 1], seed=9)
    outs = []
    for chunk, mixed in ((None, False), (6, True)):
        mr = vu.build_runner(cfg, w, dtype=dtype, device=DEV, max_total_tokens=96, max_running_requests=3,
                             chunked_prefill_size=chunk, enable_mixed_chunk=mixed)
        sch = Scheduler(mr)
        for k, p in prompts.items():
            sch.add_request(Req(k, p, SamplingParams(temperature=0, max_new_tokens=6)))
        done = sch.run_until_done()
        outs.append({k: done[k].output_ids for k in prompts})
        assert vu.pools_are_whole(mr)
    if dtype == "float32":
        for k, p in prompts.items():
            assert outs[0][k] == outs[1][k] == ref.greedy(vu.public(cfg), w, p, 6), k
    else:
        same = sum(outs[0][k] == outs[1][k] for k in prompts)
        assert same >= len(prompts) - 1


@pytest.mark.parametrize("dtype,tol", CASES)
def test_command_line_replay_of_a_model_folder(tmp_path, dtype, tol):
    """bin/trace_run as a user starts it: a model folder on disk, steps on standard input, logits in files; four live
    requests at most, a pool that the requests' total would not fit into."""
    import json
    import os
    import subprocess
    import sys

    import numpy as np

    from test_seturax_gpu import _write_model_folder

    layers = [(vu.retention(heads=2, dim=16, vdim=32, rot_dims=8, decay=(0.95, 0.999)), vu.moe(experts=4, top=2, count=2, keep=1, ff=48)),
              (vu.attention(heads=6, kv_heads=3, dim=32, rot_dims=32, base=777.0), None),
              (vu.gla(heads=4, dim=16, vdim=16, tau=2.0, rank=7), vu.moe(experts=6, top=3, count=3, keep=2, ff=24))]
    cfg = vu.make_config(layers=layers, width=64, vocab=83, groups=2, alpha=4.0, side=4)
    w = vu.make_weights(cfg, seed=17, separated_router=dtype != "float32")
    _write_model_folder(tmp_path, vu.public(cfg), w)
    prompts = vu.random_prompts(cfg, [70, 33, 1, 64, 40], seed=6)
    sched = [[("r0", 40), ("r1", 2)], [("r0", 1), ("r1", 30), ("r2", 1), ("r3", 7)], [("r0", 29), ("r1", 1), ("r3", 57)],
             [("r4", 2)], [("r4", 1)], [("r4", 37)]]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    lines, want, at = [], [], {k: 0 for k in prompts}
    full = {k: ref.forward(vu.public(cfg), w, p) for k, p in prompts.items()}
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
        assert vu.rel_err(got, expect) < tol, f"step {n}"
    assert not (out / f"{len(sched)}.f32").exists()
