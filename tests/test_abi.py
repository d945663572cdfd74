"""Host-side checks that run without a GPU: the C-ABI library loads, exports every symbol that
include/khan_aev.h declares, rejects bad arguments with status codes (never exits), and treats empty
batches as successful no-ops.  No kernel is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest

from khan_amd import _lib, datagen

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "khan_aev.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(khan_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    lib = _lib.load()
    names = declared_symbols()
    assert len(names) >= 16
    for name in names:
        assert hasattr(lib, name), "libkhan_aev.so does not export " + name
    assert set(names) == set(_lib.EXPORTED_SYMBOLS)


def test_feature_size_and_parameters():
    lib = _lib.load()
    assert lib.khan_feature_size() == 384
    r, t, a, s = ((ctypes.c_float * n)() for n in (16, 8, 4, 6))
    lib.khan_get_parameters(r, t, a, s)
    # gpu_featurizer/parameters.h:61-114
    assert list(r)[:3] == [0.5, np.float32(0.75625), np.float32(1.0125)] and r[15] == np.float32(4.34375)
    assert t[4] == np.float32(3.1415927) and list(a) == [np.float32(v) for v in (0.5, 1.15, 1.8, 2.45)]
    assert list(s) == [16.0, np.float32(4.6), np.float32(3.1), 6.0, 8.0, np.float32(0.529176917)]


def test_status_codes_without_touching_the_gpu():
    lib = _lib.load()
    assert lib.khan_status_string(0) == b"ok"
    acs0 = (ctypes.c_int32 * 4)(0, 0, 0, 0)
    acs = (ctypes.c_int32 * 4)(1, 0, 0, 0)
    n = None
    # empty batches: success, nothing launched (the reference trainer feeds them, trainer_multi_tower.py:795-817)
    assert lib.khan_featurize_f32(n, n, n, n, n, n, 0, n, n, n, n, n, acs0, n) == 0
    assert lib.khan_featurize_grad_f64(n, n, n, n, n, n, 0, n, n, n, n, n, n, n, n, acs0, n) == 0
    assert lib.khan_ani_charge_f32(n, n, n, n, n, n, 0, n, n) == 0
    assert lib.khan_mol_offsets(n, 0, 0, n, n, n) == 0
    # invalid arguments: a status code, not a crash
    assert lib.khan_featurize_f32(n, n, n, n, n, n, 1, n, n, n, n, n, acs, n) == 1
    assert lib.khan_featurize_f32(n, n, n, n, n, n, -1, n, n, n, n, n, acs, n) == 1
    assert lib.khan_featurize_f32(n, n, n, n, n, n, 1, n, n, n, n, n, None, n) == 1
    assert lib.khan_featurize_grad_f32(n, n, n, n, n, n, 1, n, n, n, n, n, n, n, n, acs, n) == 1
    assert lib.khan_ani_sort(n, 5, n, n, n, n) == 1
    assert lib.khan_ani_sort(n, -1, n, n, n, n) == 1
    assert lib.khan_ani_charge_grad_f64(n, n, n, n, n, n, 3, n, n, n) == 1
    assert lib.khan_mol_offsets(n, 1 << 40, 1, n, n, n) == 3
    # the entry points behind the networks: the sums by molecule and the dense layers
    four = (ctypes.c_void_p * 4)(None, None, None, None)
    n4 = (ctypes.c_int32 * 4)(0, 0, 0, 0)
    one4 = (ctypes.c_int32 * 4)(1, 0, 0, 0)
    assert lib.khan_mol_energy_f32(four, n, n, n, n, 0, n, n) == 0
    assert lib.khan_mol_energy_f64(four, n, n, n, n, 2, n, n) == 1
    assert lib.khan_mol_energy_f32(None, n, n, n, n, 2, n, n) == 1
    assert lib.khan_mol_energy_grad_f32(n, n, n, n, n, -1, four, n) == 1
    assert lib.khan_mol_energy_grad_f64(n, n, n, n, n, 0, four, n) == 0
    assert lib.khan_dense_f32(four, n4, 128, 128, four, None, 1, 0.1, None, four, n) == 0          # no rows: nothing to do
    assert lib.khan_dense_f32(four, one4, 128, 128, four, None, 1, 0.1, None, four, n) == 1        # rows without pointers
    assert lib.khan_dense_f32(four, n4, 100, 128, four, None, 1, 0.1, None, four, n) == 1          # width not a multiple of 32
    assert lib.khan_dense_f32(four, n4, 128, 128, four, None, 1, 0.0, None, four, n) == 1          # CELU needs alpha > 0
    assert lib.khan_dense_head_f32(four, n4, 128, 128, four, None, 1, 0.1, four, None, four, four, n) == 1   # the output layer sits behind 64 columns
    assert lib.khan_dense_head_f32(four, n4, 128, 64, four, None, 1, 0.1, four, None, four, four, n) == 0
    assert lib.khan_dense_head_grad_f32(four, four, one4, 64, 128, four, 0.1, four, four, n) == 1
    assert b"invalid" in lib.khan_status_string(1)


def test_ops_refuse_cpu_tensors():
    torch = pytest.importorskip("torch")
    from khan_amd import ops
    with pytest.raises(TypeError):
        ops.ani_sort(torch.zeros(4, dtype=torch.int32))


def test_generator_is_seeded_prefix_stable_and_physical():
    a = datagen.make_batch("organic", 200)
    b = datagen.make_batch("organic", 50)
    assert np.array_equal(a.X[:b.n_atoms], b.X) and np.array_equal(a.A[:b.n_atoms], b.A)
    c = datagen.make_batch("organic", 50, first_mol=150)
    assert np.array_equal(a.X[a.MOs[150]:], c.X)
    assert a.MACs.min() >= 3 and a.MACs.max() <= 26
    assert np.array_equal(a.MOs, np.concatenate([[0], np.cumsum(a.MACs)[:-1]]))
    xyz = np.stack([a.X, a.Y, a.Z], axis=1).astype(np.float64)
    valence = {0: 1, 1: 4, 2: 3, 3: 2}
    for m in range(a.n_mols):
        s = slice(a.MOs[m], a.MOs[m] + a.MACs[m])
        d = np.linalg.norm(xyz[s, None] - xyz[None, s], axis=-1)
        np.fill_diagonal(d, 10)
        assert d.min() >= 0.8 - 1e-6
        # hydrogens fill the valence: sum of valences is even and H count is consistent with a tree
        heavy = a.A[s][a.A[s] > 0]
        nh = int((a.A[s] == 0).sum())
        assert nh == sum(valence[int(t)] for t in heavy) - 2 * (len(heavy) - 1)
    frac = np.bincount(a.A[a.A > 0], minlength=4)[1:] / (a.A > 0).sum()
    assert abs(frac[0] - 0.6) < 0.08 and abs(frac[1] - 0.2) < 0.06
    w = b.work_counts()
    assert w["D"] == int((b.MACs.astype(np.int64) * (b.MACs - 1)).sum()) and w["C"] * 2 == w["D"]
    assert w["P_A"] <= w["P_R"] <= w["D"] and w["T"] > 0


def test_box_generator_density_and_spacing():
    b = datagen.make_batch("boxes", 3)
    assert b.MACs.min() >= 64 and b.MACs.max() <= 256
    xyz = np.stack([b.X, b.Y, b.Z], axis=1).astype(np.float64)
    for m in range(3):
        s = slice(b.MOs[m], b.MOs[m] + b.MACs[m])
        side = (b.MACs[m] / 0.1) ** (1 / 3)
        assert xyz[s].min() >= 0 and xyz[s].max() <= side + 1e-5
        d = np.linalg.norm(xyz[s, None] - xyz[None, s], axis=-1)
        np.fill_diagonal(d, 10)
        assert d.min() >= 0.9 - 1e-6


def test_normal_stream_is_position_keyed():
    full = datagen.normal(5000, 0.3, datagen.TAG_CHARGES)
    part = datagen.normal(1500, 0.3, datagen.TAG_CHARGES, first=2100)
    assert np.array_equal(full[2100:3600], part)
    assert abs(full.std() - 0.3) < 0.02 and abs(full.mean()) < 0.02


def test_build_check_of_the_lane_exchange_operand():
    """khan_amd.build.check_dpp_operands guards the one inline-asm instruction of the kernels: it has to see a
    vector write of the exchanged register within two instructions, on the fall-through path and through a
    branch, and to accept code that keeps the distance."""
    from khan_amd import build
    use = "\tv_fmac_f32_dpp v90, v2, v42 quad_perm:[0,0,0,0] row_mask:0xf bank_mask:0xf bound_ctrl:1\n"
    good = "\tds_read_b32 v2, v7\n\ts_waitcnt lgkmcnt(0)\n" + use + "\tv_mov_b32_e32 v3, v9\n\ts_nop 0\n\ts_nop 0\n" + use.replace("v2", "v3")
    assert build.check_dpp_operands(good) == 2
    with pytest.raises(RuntimeError):
        build.check_dpp_operands("\tv_mov_b32_e32 v2, v9\n\ts_nop 0\n" + use)
    with pytest.raises(RuntimeError):       # a register pair that covers the operand
        build.check_dpp_operands("\tv_lshlrev_b64 v[2:3], 1, v[8:9]\n" + use)
    with pytest.raises(RuntimeError):       # the write sits before a branch to a label just ahead of the use
        build.check_dpp_operands("\tv_mov_b32_e32 v2, v9\n\ts_branch .LBB0_7\n.LBB0_5:\n\ts_nop 0\n\ts_nop 0\n.LBB0_7:\n" + use)
    assert build.check_dpp_operands("\tv_mov_b32_e32 v90, 0\n" + use) == 1      # writing the accumulator is fine
    with pytest.raises(RuntimeError):       # the second destination of a swap
        build.check_dpp_operands("\tv_permlane32_swap_b32_e32 v88, v2\n\ts_nop 0\n" + use)
    with pytest.raises(RuntimeError):       # a vector write of EXEC needs five wait states
        build.check_dpp_operands("\tv_cmpx_gt_u32_e32 32, v0\n\ts_nop 3\n" + use)
    assert build.check_dpp_operands("\tv_cmpx_gt_u32_e32 32, v0\n\ts_nop 4\n" + use) == 1
    assert build.check_dpp_operands("\tv_mov_b32_e32 v2, v9\n\ts_nop 1\n" + use) == 1     # s_nop 1 = two wait states
    # the write sits in a block that ends in an unconditional branch elsewhere: it does not reach the use
    assert build.check_dpp_operands("\tv_mov_b32_e32 v2, v9\n\ts_branch .LBB0_9\n.LBB0_5:\n" + use) == 1


def test_the_library_cannot_be_built_without_the_lane_exchange_check():
    """build_hip() runs the check before it links, so every way of producing libkhan_aev.so goes through it."""
    import inspect
    from khan_amd import build
    src = inspect.getsource(build.build_hip)
    assert src.index("check_dpp_sources(defines)") < src.index('"-shared"')
    assert "check=" not in src and "if check" not in src          # no switch that skips it


def test_traffic_record_is_tied_to_the_kernel_sources(tmp_path, monkeypatch):
    """bench.py reports roofline.traffic from the record only while the record's digest matches the kernel sources in
    the tree; a record measured on other sources comes back as stale (bytes None), a missing one as absent."""
    import json
    import bench_profiling as profiling
    d = profiling.kernel_sources_digest()
    assert len(d) == 16 and d == profiling.kernel_sources_digest()
    rec = tmp_path / "hbm_traffic.json"
    monkeypatch.setattr(profiling, "RECORD", str(rec))
    assert profiling.measured_traffic("organic65536", "bwd") == (None, False, None)
    entry = {"bytes": 123.0, "sources_digest": d, "kernel": "k", "fetch_bytes": 100.0, "write_bytes": 23.0}
    rec.write_text(json.dumps({"organic65536/bwd": entry, "organic65536/fwd": dict(entry, sources_digest="0" * 16)}))
    b, stale, e = profiling.measured_traffic("organic65536", "bwd")
    assert (b, stale) == (123.0, False) and e["kernel"] == "k"
    b, stale, e = profiling.measured_traffic("organic65536", "fwd")
    assert b is None and stale and e is not None


def test_the_committed_traffic_record_names_the_dominant_kernels():
    """Every entry of profiles/hbm_traffic.json belongs to a (workload, pass) whose dominant kernel is known, and
    carries the pieces its total is made of."""
    import bench_profiling as profiling
    rec = profiling.load_records()
    assert rec, "profiles/hbm_traffic.json is missing or empty"
    for key, e in rec.items():
        workload, which = key.split("/")
        assert profiling.DOMINANT[(workload, which)] == e["kernel"], key
        assert abs(e["fetch_bytes"] + e["write_bytes"] - e["bytes"]) <= 1e-6 * e["bytes"]
        assert 1.9 < e["fetch_scale"] < 2.1 and 0.95 < e["write_scale"] < 1.05      # what a 64 MiB copy reads on this part


def test_measurement_builds_are_not_the_default_library(monkeypatch):
    """KHAN_AEV_LIBRARY, and nothing else, makes the package load another build of the library."""
    import importlib
    from khan_amd import build
    monkeypatch.delenv("KHAN_AEV_LIBRARY", raising=False)
    from khan_amd import _lib
    m = importlib.reload(_lib)
    assert m.LIB_PATH.endswith(os.path.join("khan_amd", "csrc", "libkhan_aev.so"))
    for k in (1, 2, 3):
        assert "stage_builds" in build.stage_variant_path(k) and build.stage_variant_path(k) != m.LIB_PATH
    monkeypatch.setenv("KHAN_AEV_LIBRARY", build.stage_variant_path(3))
    assert importlib.reload(_lib).LIB_PATH == build.stage_variant_path(3)
    monkeypatch.delenv("KHAN_AEV_LIBRARY")
    importlib.reload(_lib)


def test_library_stamp_matches_the_sources():
    """The libraries the tests load were built from the sources in the tree: the digest stamped beside each at build
    time (after the generated code passed the lane-exchange check and the link succeeded) equals the digest of the
    sources, flags and defines now.  tests/conftest.py builds again when it does not."""
    from khan_amd import build
    assert build.library_stamp() == build.sources_digest()
    assert build.library_is_current()
    assert build.library_stamp(build.CHECK_LIBRARY) == build.sources_digest(defines=build.CHECK_DEFINES)
    assert build.library_stamp() != build.library_stamp(build.CHECK_LIBRARY)
    # the digest follows the code, not the comments
    assert build._code_only("a = 1; // note\n/* more */ b = 2;") == build._code_only("a = 1;\nb = 2;")
    assert build.sources_digest(["capi.hip"]) != build.sources_digest(["charges.hip"])
