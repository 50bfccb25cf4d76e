"""bench.py contract pieces that need no GPU: more than one GPU is refused with a message, and
the algorithmic flop counts are the closed forms the roofline figures are quoted against."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2
    assert "ONE GPU" in r.stderr and r.stdout.strip() == ""


def test_algorithmic_flops_closed_forms():
    sys.path.insert(0, ROOT)
    import bench

    fl = bench.algorithmic_flops(64, 2)
    feat = 1 + 64 + 64 * 64
    assert fl["fwd"] == 4 * feat * 65 == 1081860
    assert fl["bwd"] == 2 * (2 * feat * 65 + 2 * (feat - 1) * 65 + feat * 64) == 2696068
    assert fl["build"] + fl["fwd_apply"] == fl["fwd"]
    fl1 = bench.algorithmic_flops(64, 1)
    assert fl1["fwd"] == 16900 and fl1["bwd"] == 41860
    fl32 = bench.algorithmic_flops(32, 2)
    assert fl32["fwd"] == 139524 and fl32["bwd"] == 346564


def test_executed_flops_model():
    """The executed count is pinned where it has a closed form: the d = 64 fp32 state build issues 70.5
    row-tile slots x 32 rows x 64 columns MACs per token (69 tile slots of its 23 tile waves, and the
    three Gram tiles of the remaining wave, half a slot's worth each; bf16: 72 slots), an unmasked
    consumer runs 34 slabs of 64 rows over 64 (+1 for the gradients' extra) columns, and everything
    stays below the reference-form count."""
    sys.path.insert(0, ROOT)
    import bench

    cfg = dict(B=1, H=4, N=384 * 5, D=64, mask=False, p=2, dtype="f32")
    ex = bench.executed_mfma_flops(cfg, 4)
    th = 4 * cfg["N"]
    assert ex["build_fwd"] == 2 * 70.5 * 32 * 64 * th
    assert bench.executed_mfma_flops(dict(cfg, dtype="bf16"), 4)["build_fwd"] == 2 * 72 * 32 * 64 * th
    assert ex["fwd_apply"] == ex["bwd_dv"] == 2 * 34 * 64 * 64 * th
    assert ex["bwd_dq"] == ex["bwd_dk"] == 2 * 34 * 64 * 66 * th
    al = bench.algorithmic_flops(64, 2)
    for wl in ("headline", "c4", "c2"):
        c = bench.WORKLOADS[wl]
        e = bench.executed_mfma_flops(c, c["B"] * c["H"])
        tokens = c["B"] * c["H"] * c["N"]
        f = bench.algorithmic_flops(c["D"], 2)
        assert e["build_fwd"] < f["build"] * tokens and e["fwd_apply"] < f["fwd_apply"] * tokens
        assert e["bwd_dq"] < f["bwd_dq"] * tokens and e["bwd_dv"] < f["bwd_dv"] * tokens
    # bf16 forward carries the denominator in a third accumulator tile
    cb = dict(cfg, dtype="bf16")
    assert bench.executed_mfma_flops(cb, 4)["fwd_apply"] == 2 * 34 * 64 * 96 * th


def test_executed_flops_of_the_dense_kernels():
    """Dense score tiles: 2 x 32 x 32 x d flop per contraction and (own tile, streamed tile) pair; unmasked
    every pair, causal the pairs at or below the diagonal; forward two contractions, dq three, dk/dv four."""
    sys.path.insert(0, ROOT)
    import bench

    cfg = dict(B=1, H=3, N=2048, D=64, mask=False, p=2, dtype="bf16")
    ex = bench.executed_dense_flops(cfg, 3)
    per = 2 * 32 * 32 * 64
    assert ex["fwd_apply"] == 3 * 64 * 64 * 2 * per
    assert ex["bwd_dq"] == 3 * 64 * 64 * 3 * per and ex["bwd_dk"] == 3 * 64 * 64 * 4 * per
    exm = bench.executed_dense_flops(dict(cfg, mask=True), 3)
    assert exm["fwd_apply"] == 3 * (64 * 65 // 2) * 2 * per
    # a head dimension of 48 runs as 64 padded channels, 100 tokens as 4 tiles of 32
    e48 = bench.executed_dense_flops(dict(cfg, D=48, N=100, mask=True), 1)
    assert e48["bwd_dk"] == 10 * 4 * per
    # p = 1 needs no score tile in dq
    assert bench.executed_dense_flops(dict(cfg, p=1, N=512), 3)["bwd_dq"] == 3 * 16 * 16 * 2 * per
    # p = 1 past 1024 causal / 512 unmasked positions: chunk states.  Every own tile starts from a state (one
    # 32 x d x d contraction; dk / dv two) and walks the tiles of its own 256-position chunk up to itself (1 .. 8
    # of them; unmasked none); three state builds of d x d per position
    lin = bench.executed_dense_flops(dict(cfg, p=1, mask=True), 3)
    state, walked = 2 * 32 * 64 * 64, 8 * (1 + 2 + 3 + 4 + 5 + 6 + 7 + 8)
    assert lin["fwd_apply"] == lin["bwd_dq"] == 3 * (walked * 2 * per + 64 * state)
    assert lin["bwd_dk"] == 3 * (walked * 4 * per + 64 * 2 * state)
    assert lin["build"] == 3 * 3 * 2 * 2048 * 64 * 64
    assert bench.executed_dense_flops(dict(cfg, p=1), 3)["fwd_apply"] == 3 * 64 * state


def test_traffic_figures_are_read_from_the_committed_profiles():
    """roofline.traffic is priced with the HBM bytes per token-head that the rocprofv3 summaries under
    profiles/ list for each kernel class; the summaries of both chunked workloads parse."""
    import bench

    for workload in ("headline", "c4"):
        t = bench.measured_traffic_bytes_per_token_head(workload)
        assert set(t) == {"build", "fwd_apply", "bwd_dq", "bwd_dk", "bwd_dv"}, (workload, t)
        assert all(500.0 < v < 20000.0 for v in t.values()), (workload, t)
    # the scan kernels' summaries list GiB per launch of the headline shape: four tensors of d elements per
    # token-head and kernel at least, and dq (which also reads the forward output) moves the most
    for workload, es in (("headline-p1", 4), ("headline-p1-bf16", 2)):
        t = bench.measured_traffic_bytes_per_token_head(workload)
        assert set(t) == {"fwd_apply", "bwd_dq", "bwd_dk", "bwd_dv"}, (workload, t)
        assert all(4 * 64 * es <= v < 8 * 64 * es for v in t.values()), (workload, t)
        assert max(t, key=t.get) == "bwd_dq"
    assert bench.measured_traffic_bytes_per_token_head("c2") == {}
