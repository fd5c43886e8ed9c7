"""Everything that computes the path's results, held against the committed golden vectors of tests/golden/.

The fixtures were written by tests/golden/make_golden.py from the bare definitions (index loops, math.exp in
double precision), importing neither the oracle nor the library. CPU tests here hold the oracle (numpy closed forms
and the C restatement of the reference kernel), the host model of the GPU wave programs and the C ABI's size
functions to them; the GPU tests hold the HIP path to them through the C ABI.
"""
import json
from pathlib import Path

import numpy as np
import pytest

from oracle import helix_oracle as ho

GOLDEN = Path(__file__).resolve().parent / "golden"
EXCHANGE_FIXTURES = ["exchange_c1_coded.npz", "exchange_ragged_coded.npz", "exchange_fill_vectors.npz"]
CU = 8


def load_exchange(name):
    z = np.load(GOLDEN / name, allow_pickle=False)
    cp = z["ins_o"].shape[0]
    split = lambda a: [np.ascontiguousarray(a[r]) for r in range(cp)]  # noqa: E731
    return split(z["ins_o"]), split(z["ins_s"]), split(z["outs_o"]), split(z["outs_s"])


def test_fixtures_are_what_the_generator_writes(tmp_path, monkeypatch):
    # the committed files are exactly the generator's output (no hand edits, no stale files)
    import importlib.util

    spec = importlib.util.spec_from_file_location("make_golden", GOLDEN / "make_golden.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    monkeypatch.setattr(mod, "HERE", tmp_path)
    mod.main()
    for f in EXCHANGE_FIXTURES + ["combine_small.npz"]:
        a, b = np.load(GOLDEN / f, allow_pickle=False), np.load(tmp_path / f, allow_pickle=False)
        assert sorted(a.files) == sorted(b.files)
        for k in a.files:
            assert np.array_equal(a[k], b[k], equal_nan=a[k].dtype.kind == "f"), (f, k)
    assert json.loads((GOLDEN / "sizes.json").read_text()) == json.loads((tmp_path / "sizes.json").read_text())


@pytest.mark.parametrize("name", EXCHANGE_FIXTURES)
def test_oracle_closed_forms(name):
    import torch

    ins_o, ins_s, want_o, want_s = load_exchange(name)
    for got, want in ((ho.exchange_closed_form(ins_o), want_o), (ho.exchange_closed_form(ins_s), want_s)):
        assert all(np.array_equal(g, w) for g, w in zip(got, want))
    # the torch recipes (transpose / hand-off / transpose of tests/test_alltoall.py:274-297, and the single copy)
    t_o = [torch.from_numpy(a.view(np.int16)) for a in ins_o]
    t_s = [torch.from_numpy(a.view(np.int32)) for a in ins_s]
    for fn in (ho.exchange_transpose_style, ho.exchange_single_copy):
        for got, want in ((fn(t_o), want_o), (fn(t_s), want_s)):
            assert all(np.array_equal(g.numpy().view(w.dtype), w) for g, w in zip(got, want)), fn.__name__


@pytest.mark.parametrize("name", EXCHANGE_FIXTURES)
def test_reference_kernel_model(ref_model, name):
    ins_o, ins_s, want_o, want_s = load_exchange(name)
    if (ins_o[0].shape[2] * 2) % 16 or (ins_s[0].shape[2] * 4) % 16 and ins_s[0].shape[2] != 2:
        pytest.skip("the reference's variable-width copies need 16-byte multiples (csrc/helix_alltoall.cu:115-125)")
    cp = len(ins_o)
    ws = ref_model.new_workspace(cp, 132)
    got_o, got_s = ref_model.alltoall_all_ranks(ins_o, ins_s, ws, sm_count=132)
    for r in range(cp):
        assert np.array_equal(got_o[r], want_o[r]) and np.array_equal(got_s[r], want_s[r])


@pytest.mark.parametrize("channels", [1, 3])
@pytest.mark.parametrize("name", EXCHANGE_FIXTURES)
def test_host_model_of_the_wave_programs(host_model, name, channels):
    ins_o, ins_s, want_o, want_s = load_exchange(name)
    cp = len(ins_o)
    ws = host_model.new_workspace(cp, CU)
    got_o, got_s, rc, msg = host_model.alltoall(ins_o, ins_s, ws, CU, channels)
    assert rc == 0, msg
    for r in range(cp):
        assert np.array_equal(got_o[r], want_o[r]) and np.array_equal(got_s[r], want_s[r])


def test_oracle_combine():
    z = np.load(GOLDEN / "combine_small.npz", allow_pickle=False)
    got, got_lse = ho.lse_combine(z["outputs"], z["lses"], dtype=np.float64)
    assert np.allclose(got, z["combined"], rtol=1e-12, atol=1e-15)
    assert np.array_equal(np.isneginf(got_lse), np.isneginf(z["global_lse"]))
    fin = np.isfinite(z["global_lse"])
    assert np.allclose(got_lse[fin], z["global_lse"][fin], rtol=1e-12, atol=1e-12)
    # float32 evaluation, the precision the device works in
    got32, _ = ho.lse_combine(z["outputs"], z["lses"], dtype=np.float32)
    assert np.allclose(got32, z["combined"], rtol=1e-5, atol=1e-6)


def test_sizes(ref_model):
    from helix_a2a import _ops

    doc = json.loads((GOLDEN / "sizes.json").read_text())
    for row in doc["table"]:
        cp, units = row["cp"], row["units"]
        assert ho.max_channel_count(cp, units) == row["max_channels"]
        assert ho.workspace_size(cp, units) == row["workspace_bytes"]
        assert ref_model.workspace_size(cp, units) == row["workspace_bytes"]
        assert _ops.max_channel_count(cp, units) == row["max_channels"]          # the C ABI, no device involved
        assert _ops.get_workspace_size_per_rank(cp, units) == row["workspace_bytes"]
    known = doc["known"]
    assert _ops.get_workspace_size_per_rank(8, 256) == known["cp8_256cu"]
    assert _ops.get_workspace_size_per_rank(4, 256) == known["cp4_256cu"]
    assert _ops.get_workspace_size_per_rank(2, 256) == known["cp2_256cu"]
    assert _ops.get_workspace_size_per_rank(16, 256) == known["cp16_256cu"]
    assert _ops.get_workspace_size_per_rank(8, 132) == known["cp8_132sm"]


# ---------------------------------------------------------------------------
# the HIP path
# ---------------------------------------------------------------------------

@pytest.fixture(scope="module")
def hx():
    import torch

    import helix_a2a

    assert torch.cuda.is_available()
    return helix_a2a


_WS = {}


def _workspace(hx, cp):
    if cp not in _WS:
        _WS[cp] = hx.allocate_workspace(cp, 0)
        for r in range(cp):
            hx.init_workspace(_WS[cp], r, cp)
    return _WS[cp]


@pytest.mark.gpu
@pytest.mark.parametrize("channels", [0, 1])
@pytest.mark.parametrize("name", EXCHANGE_FIXTURES)
def test_gpu_exchange(hx, name, channels):
    import torch

    ins_o, ins_s, want_o, want_s = load_exchange(name)
    cp = len(ins_o)
    ws = _workspace(hx, cp)
    dev_o = [torch.from_numpy(a.view(np.int16)).view(torch.bfloat16).cuda() for a in ins_o]
    dev_s = [torch.from_numpy(a.view(np.int32)).view(torch.float32).cuda() for a in ins_s]
    got_o, got_s = hx.alltoall_loopback(dev_o, dev_s, ws, channel_count=channels)
    per_rank = [hx.alltoall(dev_o[r], dev_s[r], ws, cp_rank=r, cp_size=cp) for r in range(cp)]
    torch.cuda.synchronize()
    for r in range(cp):
        assert np.array_equal(ho.torch_bits(got_o[r]), want_o[r]) and np.array_equal(ho.torch_bits(got_s[r]), want_s[r])
        assert np.array_equal(ho.torch_bits(per_rank[r][0]), want_o[r])
        assert np.array_equal(ho.torch_bits(per_rank[r][1]), want_s[r])
    from helix_a2a import _ops
    assert _ops.device_status() == 0


@pytest.mark.gpu
def test_gpu_combine(hx):
    import torch

    z = np.load(GOLDEN / "combine_small.npz", allow_pickle=False)
    outputs, lses, want, want_lse = z["outputs"], z["lses"], z["combined"], z["global_lse"]
    n, b, h, d = outputs.shape
    ws = _workspace(hx, n)
    # rank s holds [B, n*h, D]: head group r of every rank carries the fixture's shard s (the same for all r)
    outs = [torch.from_numpy(np.tile(outputs[s], (1, n, 1))).to(torch.bfloat16).cuda() for s in range(n)]
    ls = [torch.from_numpy(np.tile(lses[s], (1, n))).cuda() for s in range(n)]
    assert all(torch.equal(o.float().cpu(), torch.from_numpy(np.tile(outputs[s], (1, n, 1)))) for s, o in enumerate(outs))
    got, got_lse = hx.dcp_a2a_lse_reduce(outs, ls, ws, return_lse=True)
    torch.cuda.synchronize()
    for r in range(n):
        g = got[r].float().cpu().numpy()
        assert (np.abs(g - want) <= 2e-2 + 2e-2 * np.abs(want)).all(), f"rank {r}: off by {np.abs(g - want).max()}"
        gl = got_lse[r].cpu().numpy()
        assert np.array_equal(np.isneginf(gl), np.isneginf(want_lse))
        fin = np.isfinite(want_lse)
        assert np.allclose(gl[fin], want_lse[fin], atol=1e-4)
    from helix_a2a import _ops
    assert _ops.device_status() == 0
