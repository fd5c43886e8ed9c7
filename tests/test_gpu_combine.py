"""GPU tests of the exchange fused with the LSE-weighted combine, against the oracle.

Tolerance: 2e-2 absolute plus 2e-2 relative on the bf16/fp16 result (the oracle
reduces in fp32 and does not round its result); the combined log-sum-exp is
fp32 on both sides and is held to 1e-4.
"""
import numpy as np
import pytest
import torch

from helix_testing import torch_bits
from oracle import helix_oracle as ho

pytestmark = pytest.mark.gpu

ATOL = RTOL = 2e-2


@pytest.fixture(scope="module")
def hx():
    import helix_a2a

    assert torch.cuda.is_available()
    return helix_a2a


@pytest.fixture(scope="module")
def ops(hx):
    from helix_a2a import _ops

    return _ops


_WS = {}


def workspace(hx, cp):
    ws = _WS.get(cp)
    if ws is None:
        ws = _WS[cp] = hx.allocate_workspace(cp, 0)
        for r in range(cp):
            hx.init_workspace(ws, r, cp)
    return ws


def oracle_combine(ins_o, ins_s, heads, mode, widen):
    """Exchange (closed form on bits) followed by the reference's combine, per rank."""
    recv_o = ho.exchange_closed_form([torch_bits(t) for t in ins_o])
    recv_s = ho.exchange_closed_form([torch_bits(t) for t in ins_s])
    out = []
    for r in range(len(ins_o)):
        o32 = widen(recv_o[r])
        s32 = recv_s[r].view(np.float32)
        with np.errstate(all="ignore"):
            out.append(ho.combine_after_exchange(o32, s32, heads, mode))
    return out


def check(combined, lse, want, dtype):
    for r, (want_c, want_l) in enumerate(want):
        got = combined[r].float().cpu().numpy().reshape(want_c.shape)
        finite = np.isfinite(want_c)
        assert np.array_equal(np.isfinite(got), finite), f"rank {r}: non-finite pattern differs"
        err = np.abs(got[finite] - want_c[finite])
        bound = ATOL + RTOL * np.abs(want_c[finite])
        assert (err <= bound).all(), f"rank {r}: max error {err.max()} (dtype {dtype})"
        if lse is not None:
            g = lse[r].cpu().numpy()
            inf = np.isneginf(want_l)
            assert np.array_equal(np.isneginf(g), inf)
            assert np.allclose(g[~inf], want_l[~inf], rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("name", ["c1", "c2", "c5b", "c3", "c4", "c5a"])
def test_combine_workloads(hx, ops, name):
    from helix_workloads import WORKLOADS, make_inputs

    w = WORKLOADS[name]
    ws = workspace(hx, w.cp)
    ins_o, ins_s = make_inputs(w, "cuda")
    combined, lse = hx.alltoall_combine_loopback(ins_o, ins_s, ws, hx.STATS_MAX_SUM, return_lse=True)
    torch.cuda.synchronize()
    assert ops.device_status() == 0
    assert combined[0].shape == (w.tokens, w.heads_per_rank * w.head_dim) and lse[0].shape == (w.tokens, w.heads_per_rank)
    want = oracle_combine(ins_o, ins_s, w.heads_per_rank, 1, ho.bf16_bits_to_f32)
    check(combined, lse, want, "bf16")


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_combine_modes_dtypes_and_masked_heads(hx, ops, mode, dtype):
    cp, tokens, heads, d = 4, 19, 3, 64
    ws = workspace(hx, cp)
    g = torch.Generator().manual_seed(mode * 2 + (dtype == torch.float16))
    ins_o = [torch.randn(tokens, cp, heads * d, generator=g).to(dtype).cuda() for _ in range(cp)]
    ins_s = []
    for r in range(cp):
        mx = torch.randn(tokens, cp, heads, generator=g) * 3
        sm = 1 + torch.rand(tokens, cp, heads, generator=g) * 100
        mx[torch.rand(tokens, cp, heads, generator=g) < 0.2] = float("-inf")  # fully masked shards
        if r == 1:
            mx[0] = float("-inf")  # a whole token masked on one rank
        ins_s.append(torch.stack((mx, sm), -1).reshape(tokens, cp, 2 * heads).contiguous().cuda())
    for t in ins_s:
        t[1] = torch.where(torch.arange(2 * heads, device="cuda") % 2 == 0, float("-inf"), 1.0)  # every shard masked
    ins_s[2][3, :, 0] = float("nan")   # NaN and +inf statistics count as masked
    ins_s[3][4, :, 0] = float("inf")
    combined, lse = hx.alltoall_combine_loopback(ins_o, ins_s, ws, mode, return_lse=True)
    torch.cuda.synchronize()
    assert ops.device_status() == 0
    widen = ho.bf16_bits_to_f32 if dtype == torch.bfloat16 else ho.f16_bits_to_f32
    want = oracle_combine(ins_o, ins_s, heads, mode, widen)
    check(combined, lse, want, str(dtype))
    for r in range(cp):
        assert bool((combined[r][1] == 0).all()), "a head masked on every rank combines to zero"


def test_combine_closed_forms(hx, ops):
    # equal statistics -> arithmetic mean of the partial outputs; one dominant shard -> that shard
    cp, tokens, heads, d = 8, 5, 2, 128
    ws = workspace(hx, cp)
    g = torch.Generator().manual_seed(3)
    ins_o = [torch.randn(tokens, cp, heads * d, generator=g).to(torch.bfloat16).cuda() for _ in range(cp)]
    equal = [torch.tensor([0.5, 7.0]).repeat(tokens, cp, heads).cuda() for _ in range(cp)]
    combined = hx.alltoall_combine_loopback(ins_o, equal, ws, hx.STATS_MAX_SUM)
    torch.cuda.synchronize()
    for r in range(cp):
        mean = torch.stack([ins_o[s][:, r, :].float() for s in range(cp)]).mean(0)
        assert torch.allclose(combined[r].float(), mean, atol=ATOL, rtol=RTOL)
    dominant = []
    for s in range(cp):
        lse = torch.full((tokens, cp, heads), 0.0 if s != 5 else 60.0)
        dominant.append(torch.stack((lse, torch.zeros_like(lse)), -1).reshape(tokens, cp, 2 * heads).contiguous().cuda())
    combined, lse = hx.alltoall_combine_loopback(ins_o, dominant, ws, hx.STATS_LSE, return_lse=True)
    torch.cuda.synchronize()
    assert ops.device_status() == 0
    for r in range(cp):
        assert torch.equal(combined[r], ins_o[5][:, r, :])      # weight 1 up to e^-60: bit-exact pass-through
        assert torch.allclose(lse[r], torch.full_like(lse[r], 60.0))


def test_combine_4d_inputs_and_plan_replay(hx, ops):
    from helix_workloads import WORKLOADS, make_inputs

    w = WORKLOADS["c2"]
    ws = workspace(hx, w.cp)
    ins_o, ins_s = make_inputs(w, "cuda")
    hp = w.heads_per_rank
    o4 = [t.view(w.tokens, w.cp, hp, w.head_dim) for t in ins_o]
    s4 = [t.view(w.tokens, w.cp, hp, 2) for t in ins_s]
    plan = ops.CombinePlan(o4, s4, ws, ops.STATS_MAX_SUM, return_lse=False, channel_count=16)
    want = oracle_combine(ins_o, ins_s, hp, 1, ho.bf16_bits_to_f32)
    for _ in range(6):  # replays walk through the FIFO entries
        combined = plan.run()
    torch.cuda.synchronize()
    assert ops.device_status() == 0
    assert combined[0].shape == (w.tokens, hp, w.head_dim)
    check(combined, None, want, "bf16")


def test_combine_serves_at_most_thirty_two_ranks(hx, ops):
    cp = 33
    ws = torch.zeros(cp, 8, dtype=torch.int64, device="cuda")  # never reached: the rank count is checked first
    o = [torch.zeros(1, cp, 64, dtype=torch.bfloat16, device="cuda") for _ in range(cp)]
    s = [torch.zeros(1, cp, 2, device="cuda") for _ in range(cp)]
    with pytest.raises(RuntimeError, match="at most 32 ranks"):
        hx.alltoall_combine_loopback(o, s, ws, hx.STATS_LSE)
    with pytest.raises(RuntimeError, match="at most 32 ranks"):
        hx.dcp_a2a_lse_reduce([torch.zeros(1, 66, 32, dtype=torch.bfloat16, device="cuda")] * cp,
                              [torch.zeros(1, 66, device="cuda")] * cp, ws)


def test_combine_rejects_bad_shapes(hx, ops):
    cp = 2
    ws = workspace(hx, cp)
    o = [torch.zeros(2, cp, 72, dtype=torch.bfloat16, device="cuda") for _ in range(cp)]   # 72 elements, 4 heads -> head_dim 18
    s = [torch.zeros(2, cp, 8, device="cuda") for _ in range(cp)]
    with pytest.raises(RuntimeError, match="head_dim"):
        hx.alltoall_combine_loopback(o, s, ws)
    with pytest.raises(RuntimeError, match="stats_mode"):
        hx.alltoall_combine_loopback(o, s, ws, stats_mode=7)


def test_combine_large_messages_many_ranks(hx, ops):
    # 16 ranks x 16.5 KB messages, head_dim 96: units straddle head boundaries (96 * 2 / 8 = 24 pieces per head)
    cp, tokens, heads, d = 16, 3, 4, 96
    ws = workspace(hx, cp)
    g = torch.Generator().manual_seed(11)
    ins_o = [torch.randn(tokens, cp, heads * d, generator=g).to(torch.bfloat16).cuda() for _ in range(cp)]
    ins_s = [torch.stack((torch.randn(tokens, cp, heads, generator=g) * 2,
                          1 + torch.rand(tokens, cp, heads, generator=g) * 50), -1)
             .reshape(tokens, cp, 2 * heads).contiguous().cuda() for _ in range(cp)]
    combined, lse = hx.alltoall_combine_loopback(ins_o, ins_s, ws, hx.STATS_MAX_SUM, return_lse=True)
    torch.cuda.synchronize()
    assert ops.device_status() == 0
    check(combined, lse, oracle_combine(ins_o, ins_s, heads, 1, ho.bf16_bits_to_f32), "bf16")
    big_o = [torch.randn(2, cp, 8192, generator=g).to(torch.bfloat16).cuda() for _ in range(cp)]
    big_s = [torch.rand(2, cp, 32, generator=g).cuda() + 0.5 for _ in range(cp)]
    combined = hx.alltoall_combine_loopback(big_o, big_s, ws, hx.STATS_LSE)
    torch.cuda.synchronize()
    assert ops.device_status() == 0
    check(combined, None, oracle_combine(big_o, big_s, 16, 0, ho.bf16_bits_to_f32), "bf16")


@pytest.mark.parametrize("cp", [3, 6, 12, 24])
@pytest.mark.parametrize("tokens", [1, 3, 5, 7, 9, 11, 33])
def test_combine_every_units_in_flight_variant(hx, ops, cp, tokens):
    # one channel, 2 heads x 128 + 2 pairs of statistics = 528 bytes = 66 pieces = 4.4 lines per message: the run
    # of `tokens` messages selects the sender program with 1, 2, ... 6 units in flight per lane, and the four
    # rank counts select the 4-, 8-, 16- and 32-lanes-per-slot combine kernels
    heads, d = 2, 128
    ws = workspace(hx, cp)
    g = torch.Generator().manual_seed(100 * cp + tokens)
    ins_o = [torch.randn(tokens, cp, heads * d, generator=g).to(torch.bfloat16).cuda() for _ in range(cp)]
    ins_s = [torch.stack((torch.randn(tokens, cp, heads, generator=g) * 2,
                          1 + torch.rand(tokens, cp, heads, generator=g) * 50), -1)
             .reshape(tokens, cp, 2 * heads).contiguous().cuda() for _ in range(cp)]
    combined, lse = hx.alltoall_combine_loopback(ins_o, ins_s, ws, hx.STATS_MAX_SUM, return_lse=True, channel_count=1)
    torch.cuda.synchronize()
    assert ops.device_status() == 0
    check(combined, lse, oracle_combine(ins_o, ins_s, heads, 1, ho.bf16_bits_to_f32), "bf16")


def test_combine_beyond_fifo_capacity_runs_in_rounds(hx, ops):
    # one channel, 66-piece messages: 232 per FIFO entry, 928 per round of four entries; 2000 tokens take three rounds
    cp, tokens, heads, d = 2, 2000, 2, 128
    ws = workspace(hx, cp)
    g = torch.Generator().manual_seed(41)
    ins_o = [torch.randn(tokens, cp, heads * d, generator=g).to(torch.bfloat16).cuda() for _ in range(cp)]
    ins_s = [torch.stack((torch.randn(tokens, cp, heads, generator=g) * 2,
                          1 + torch.rand(tokens, cp, heads, generator=g) * 50), -1)
             .reshape(tokens, cp, 2 * heads).contiguous().cuda() for _ in range(cp)]
    want = oracle_combine(ins_o, ins_s, heads, 1, ho.bf16_bits_to_f32)
    for _ in range(2):          # twice: the step counters continue from where the rounds left them
        combined, lse = hx.alltoall_combine_loopback(ins_o, ins_s, ws, hx.STATS_MAX_SUM, return_lse=True, channel_count=1)
        torch.cuda.synchronize()
        assert ops.device_status() == 0
        check(combined, lse, want, "bf16")


def test_combine_thirty_two_ranks(hx, ops):
    # the largest rank count: 32 senders per (message, head), two slots per sideways pass
    cp, tokens, heads, d = 32, 20, 2, 64
    ws = workspace(hx, cp)
    g = torch.Generator().manual_seed(32)
    ins_o = [torch.randn(tokens, cp, heads * d, generator=g).to(torch.bfloat16).cuda() for _ in range(cp)]
    ins_s = [torch.stack((torch.randn(tokens, cp, heads, generator=g) * 2,
                          1 + torch.rand(tokens, cp, heads, generator=g) * 50), -1)
             .reshape(tokens, cp, 2 * heads).contiguous().cuda() for _ in range(cp)]
    ins_s[5][3, 7, 0] = float("-inf")      # one sender masked for one head
    for channels in (0, 3):
        combined, lse = hx.alltoall_combine_loopback(ins_o, ins_s, ws, hx.STATS_MAX_SUM, return_lse=True,
                                                     channel_count=channels)
        torch.cuda.synchronize()
        assert ops.device_status() == 0
        check(combined, lse, oracle_combine(ins_o, ins_s, heads, 1, ho.bf16_bits_to_f32), "bf16")


def test_combine_while_senders_are_still_writing(hx, ops):
    # few channels: all wavefronts resident at once, the combine half has to wait for its senders
    from helix_workloads import WORKLOADS, make_inputs

    w = WORKLOADS["c3"]
    ws = workspace(hx, w.cp)
    ins_o, ins_s = make_inputs(w, "cuda")
    want = oracle_combine(ins_o, ins_s, w.heads_per_rank, 1, ho.bf16_bits_to_f32)
    for channels in (4, 8, 16):
        plan = ops.CombinePlan(ins_o, ins_s, ws, ops.STATS_MAX_SUM, return_lse=True, channel_count=channels)
        first = None
        for it in range(40):
            combined, lse = plan.run()
            if first is None:
                torch.cuda.synchronize()
                check(combined, lse, want, "bf16")
                first = [c.clone() for c in combined]
            else:
                for r in range(w.cp):  # the reduction order is fixed: every replay gives the same bits
                    assert torch.equal(combined[r], first[r]), f"replay {it} differs on rank {r} with {channels} channels"
    torch.cuda.synchronize()
    assert ops.device_status() == 0


@pytest.mark.parametrize("base_e", [True, False])
def test_dcp_a2a_lse_reduce_matches_the_reference_recipe(hx, ops, base_e):
    # What the serving integration computes (patches/dcp_alltoall_helix.py:455-504): every rank splits its
    # [B, H, D] output by head group, the groups are exchanged, and each rank combines its N partials.
    n, b, h, d = 8, 33, 64, 128
    ws = workspace(hx, n)
    g = torch.Generator().manual_seed(21)
    outs = [torch.randn(b, h, d, generator=g).to(torch.bfloat16).cuda() for _ in range(n)]
    lses = [(torch.randn(b, h, generator=g) * 4).cuda() for _ in range(n)]
    lses[3][5, 7] = float("-inf")
    combined, glse = hx.dcp_a2a_lse_reduce(outs, lses, ws, return_lse=True, is_lse_base_on_e=base_e)
    torch.cuda.synchronize()
    assert ops.device_status() == 0
    hp = h // n
    assert combined[0].shape == (b, hp, d) and glse[0].shape == (b, hp)
    o32 = np.stack([ho.bf16_bits_to_f32(torch_bits(t)) for t in outs])          # [N, B, H, D]
    l32 = np.stack([t.cpu().numpy() for t in lses])                               # [N, B, H]
    if not base_e:
        l32 = l32 * np.float32(np.log(2.0))
    for r in range(n):
        with np.errstate(all="ignore"):
            want, want_lse = ho.lse_combine(o32[:, :, r * hp:(r + 1) * hp, :], l32[:, :, r * hp:(r + 1) * hp])
        if not base_e:
            want_lse = want_lse / np.float32(np.log(2.0))
        got = combined[r].float().cpu().numpy()
        assert (np.abs(got - want) <= ATOL + RTOL * np.abs(want)).all()
        assert np.allclose(glse[r].cpu().numpy(), want_lse, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("n,h,d,base_e", [
    (16, 16, 128, True),    # the 16-head MLA model of the reference's benchmark at N = 16: one head per rank
    (4, 12, 64, True),      # three heads per rank
    (4, 12, 64, False),     # ... with base-2 log-sum-exps
    (8, 8, 576, False),     # one head per rank, MLA width (512 + 64), base 2
    (2, 10, 32, True),      # five heads per rank, the smallest head
    (3, 3, 96, True),       # one head per rank, three ranks
])
def test_dcp_a2a_lse_reduce_any_heads_per_rank(hx, ops, n, h, d, base_e):
    # H/N need not be even: the reference pads every LSE to a pair (patches/dcp_alltoall_helix.py:560-567),
    # here a row of H/N floats travels as it is; and the base of the logarithms is taken inside the kernel
    b = 19
    ws = workspace(hx, n)
    g = torch.Generator().manual_seed(1000 * n + h)
    outs = [torch.randn(b, h, d, generator=g).to(torch.bfloat16).cuda() for _ in range(n)]
    lses = [(torch.randn(b, h, generator=g) * 3).cuda() for _ in range(n)]
    lses[0][2, h - 1] = float("-inf")
    lses[n - 1][b - 1, 0] = float("nan")
    hp = h // n
    o32 = np.stack([ho.bf16_bits_to_f32(torch_bits(t)) for t in outs])          # [N, B, H, D]
    l32 = np.stack([t.cpu().numpy() for t in lses])                               # [N, B, H]
    if not base_e:
        l32 = l32 * np.float32(np.log(2.0))
    for _ in range(2):   # the second call finds the descriptors of the shape cached
        combined, glse = hx.dcp_a2a_lse_reduce(outs, lses, ws, return_lse=True, is_lse_base_on_e=base_e)
        torch.cuda.synchronize()
        assert ops.device_status() == 0
        assert combined[0].shape == (b, hp, d) and glse[0].shape == (b, hp)
        for r in range(n):
            with np.errstate(all="ignore"):
                want, want_lse = ho.lse_combine(o32[:, :, r * hp:(r + 1) * hp, :], l32[:, :, r * hp:(r + 1) * hp])
            if not base_e:
                want_lse = want_lse / np.float32(np.log(2.0))
            got = combined[r].float().cpu().numpy()
            assert (np.abs(got - want) <= ATOL + RTOL * np.abs(want)).all(), f"rank {r}"
            assert np.allclose(glse[r].cpu().numpy(), want_lse, rtol=1e-4, atol=1e-4), f"rank {r}"
    # without the combined LSE
    only = hx.dcp_a2a_lse_reduce(outs, lses, ws, is_lse_base_on_e=base_e)
    torch.cuda.synchronize()
    for r in range(n):
        assert torch.equal(only[r], combined[r])


# ---------------------------------------------------------------------------
# the pipeline benchmark's three formulations agree, eagerly and from captured graphs
# ---------------------------------------------------------------------------

def _load_pipeline_benchmark():
    import importlib.util
    import os

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "helix-a2a_amd", "benchmark",
                        "benchmark_helix_pipeline.py")
    spec = importlib.util.spec_from_file_location("benchmark_helix_pipeline", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_pipeline_benchmark_formulations_agree(hx, ops):
    pb = _load_pipeline_benchmark()
    n, b, h, d = 4, 16, 32, 128
    ws = workspace(hx, n)
    g = torch.Generator().manual_seed(77)
    outs = [torch.randn(b, h, d, generator=g).to(torch.bfloat16).cuda() for _ in range(n)]
    lses = [(torch.randn(b, h, generator=g).abs() + 1.0).cuda() for _ in range(n)]
    lses[1][3, 5] = float("-inf")                      # a masked shard
    # the benchmark's torch combine against the oracle's fp64 combine
    want = ho.lse_combine(np.stack([ho.bf16_bits_to_f32(torch_bits(o)) for o in outs]),
                          np.stack([l.cpu().numpy() for l in lses]), dtype=np.float64)[0]    # [B, H, D]
    off = pb.Stages(False)
    for name in ("dcp", "recipe", "fused"):
        got = pb.PIPELINES[name](outs, lses, ws, off)
        torch.cuda.synchronize()
        for r in range(n):
            ref = want[:, r * (h // n):(r + 1) * (h // n), :]
            err = np.abs(got[r].float().cpu().numpy() - ref)
            assert (err <= 2e-2 + 2e-2 * np.abs(ref)).all(), f"{name}: rank {r} off by {err.max()}"
    # each pipeline replays from a captured graph and the timer returns sane figures
    for name in ("recipe", "fused"):
        res = pb.bench_graph(pb.PIPELINES[name], outs, lses, ws, warmup=2, iters=5)
        assert 0 < res["total"]["p50"] < 1e5
    res = pb.bench_eager(pb.pipeline_recipe, outs, lses, ws, warmup=1, iters=3)
    assert set(res) == {"total", "copy", "a2a", "combine"}
    assert ops.device_status() == 0


def test_dcp_a2a_lse_reduce_argument_checks_and_descriptor_reuse(hx, ops):
    n, b, h, d = 4, 5, 8, 64
    ws = workspace(hx, n)
    g = torch.Generator().manual_seed(5)

    def make(bb=b, hh=h, dd=d, dtype=torch.bfloat16):
        return ([torch.randn(bb, hh, dd, generator=g).to(dtype).cuda() for _ in range(n)],
                [torch.randn(bb, hh, generator=g).cuda() for _ in range(n)])

    outs, lses = make()
    bad = [
        (outs[:3], lses, "one attention output"),                                   # rank count mismatch
        ([o.float() for o in outs], lses, "half or bfloat16"),
        ([o.cpu() for o in outs], lses, "GPU"),
        (outs, [l.double() for l in lses], "float32"),
        (outs[:3] + [outs[3][:, :4]], lses, "one shape"),
        (make(hh=6)[0], make(hh=6)[1], "divisible"),
        (make(dd=16)[0], make(dd=16)[1], "head_dim"),
    ]
    for o, l, pattern in bad:
        with pytest.raises(RuntimeError, match=pattern):
            hx.dcp_a2a_lse_reduce(o, l, ws)
    # the cached descriptor arrays of a shape serve fresh tensors on every call
    for _ in range(3):
        outs, lses = make()
        got, got_lse = hx.dcp_a2a_lse_reduce(outs, lses, ws, return_lse=True)
        torch.cuda.synchronize()
        want, want_lse = ho.lse_combine(np.stack([ho.bf16_bits_to_f32(torch_bits(o)) for o in outs]),
                                        np.stack([l.cpu().numpy() for l in lses]), dtype=np.float64)
        for r in range(n):
            ref = want[:, r * (h // n):(r + 1) * (h // n), :]
            assert (np.abs(got[r].float().cpu().numpy() - ref) <= ATOL + RTOL * np.abs(ref)).all()
            assert np.allclose(got_lse[r].cpu().numpy(), want_lse[:, r * (h // n):(r + 1) * (h // n)], atol=1e-4)
    # an empty batch launches nothing
    e_o, e_l = make(bb=0)
    assert all(t.shape == (0, h // n, d) for t in hx.dcp_a2a_lse_reduce(e_o, e_l, ws))
    assert ops.device_status() == 0
