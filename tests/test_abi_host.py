"""The C-ABI library loads, exports every symbol the header declares, and rejects bad
arguments on the host (no kernel is launched here: runs without a GPU)."""
import ctypes as C
import os
import re

import pytest
import torch

from conftest import ROOT

import fastgl
from fastgl import _lib as L


def _declared():
    text = open(os.path.join(ROOT, "include", "fastgl_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fgl_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared()
    assert len(names) >= 20
    raw = C.CDLL(L.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), n
    assert sorted(L.SIGNATURES) == names  # the python binding covers the header, nothing else


def test_pure_host_entry_points():
    lib = fastgl.lib()
    assert lib.fgl_abi_version() == 11
    assert fastgl.table_size(40960, 2) == 131072
    assert fastgl.table_size(8110080, 2) == 16777216
    assert lib.fgl_idmap_slots(0) == 64 and lib.fgl_idmap_slots(33) == 128 and lib.fgl_idmap_slots(8650752) == 1 << 25
    assert lib.fgl_idmap_table_bytes(1 << 25) == 8 << 25
    assert lib.fgl_exclusive_sum_workspace_bytes(10) > 0
    # the host side of a read-back, where no device is involved: words that are there already, and bad arguments
    words = (C.c_int32 * 3)(5, 0, 7)
    assert lib.fgl_wait_words(words, 3, -1, None, 1000) == 0
    assert lib.fgl_wait_words(words, 0, -1, None, 1000) != 0 and lib.fgl_wait_words(None, 3, -1, None, 1000) != 0


def test_static_scratch_holds_the_workspace_of_its_largest_call():
    # fgl_sample_node_static's 16 MiB array against what the workspace formula asks for at the stated seed limit
    lib = fastgl.lib()
    text = open(os.path.join(ROOT, "include", "fastgl_hip.h")).read()
    max_seeds = int(re.search(r"#define FGL_STATIC_MAX_SEEDS (\d+)", text).group(1))
    assert max_seeds == 1 << 20
    for fanout in (1, 48, 49, L.MAX_FANOUT):
        assert 0 < lib.fgl_sample_workspace_bytes(max_seeds, fanout) <= 16 << 20


def test_plan_matches_the_worst_case_table():
    # batch 8192, hops expanded with 5, 10, 15 on the 111M-node graph
    fan = (C.c_int32 * 3)(5, 10, 15)
    cd, ce = (C.c_int64 * 3)(), (C.c_int64 * 3)()
    cu, sl, ws = C.c_int64(), C.c_int64(), C.c_size_t()
    L.check(fastgl.lib().fgl_sample_blocks_plan(111_000_000, 8192, fan, 3, None, 0, cd, ce, C.byref(cu), C.byref(sl), C.byref(ws)))
    assert list(cd) == [8192, 49152, 540672]
    assert list(ce) == [40960, 491520, 8110080]
    assert cu.value == 8650752 and sl.value == 1 << 25 and ws.value > 0
    # a small graph caps the bounds
    L.check(fastgl.lib().fgl_sample_blocks_plan(1000, 100, fan, 3, None, 0, cd, ce, C.byref(cu), C.byref(sl), C.byref(ws)))
    assert list(cd) == [100, 600, 1100] and cu.value == 1100
    # the caller's own limits clip the plan
    lim = (C.c_int64 * 4)(100, 300, 400, 500)
    L.check(fastgl.lib().fgl_sample_blocks_plan(111_000_000, 100, fan, 3, lim, 0, cd, ce, C.byref(cu), C.byref(sl), C.byref(ws)))
    assert list(cd) == [100, 300, 400] and list(ce) == [500, 3000, 6000] and cu.value == 500
    bad = (C.c_int64 * 4)(50, 300, 400, 500)
    assert fastgl.lib().fgl_sample_blocks_plan(111_000_000, 100, fan, 3, bad, 0, cd, ce, C.byref(cu), C.byref(sl), C.byref(ws)) == 1
    # limits that shrink from one hop to the next are refused (a hop's nodes are a prefix of the next hop's)
    shrinking = (C.c_int64 * 4)(100, 400, 300, 500)
    assert fastgl.lib().fgl_sample_blocks_plan(111_000_000, 100, fan, 3, shrinking, 0, cd, ce, C.byref(cu), C.byref(sl), C.byref(ws)) == 1
    assert b"below an earlier entry" in fastgl.lib().fgl_last_error()


def test_argument_errors_are_reported_not_launched():
    lib = fastgl.lib()
    fan = (C.c_int32 * 1)(0)
    assert lib.fgl_sample_blocks_plan(10, 10, fan, 1, None, 0, None, None, None, None, None) == 1
    assert b"fanout" in lib.fgl_last_error()
    assert lib.fgl_sample_node(None, 1, None, 10, None, 5, None, 500, 0, 0, None, None, None, None, None, None, None, 0, None) == 1
    assert lib.fgl_idmap_reset(None, 100, None) == 1      # not a power of two / null table
    assert lib.fgl_aggregate(None, None, 4, None, None, 8, 8, 7, 0, 0, None, None, None, 1, None, -1, None, -1, None, 8, None) == 1
    assert b"dtype" in lib.fgl_last_error()
    assert lib.fgl_rmat_keys(0, 10, 40, 100, 0, None, None) == 1
    # the entry point with the library's own scratch states its limit before touching the GPU
    assert lib.fgl_sample_node_static(None, 1, None, 10, None, (1 << 20) + 1, None, 5, 0, 0, None, None, None, None, None, None) == 1
    assert b"1048576" in lib.fgl_last_error()


def test_operator_input_checks_raise_runtime_error():
    cpu = torch.zeros(4, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        fastgl.cal_deg(cpu, 4)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        fastgl.sample_node(cpu, cpu, cpu, cpu, 4, 2)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        fastgl.transfer_edge_id(cpu, cpu, cpu, 4, 8, 4, 4)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        fastgl.forward_gat(cpu, torch.zeros(4, 2), cpu, torch.zeros(4, 4), 2, 4, 2)


def test_sampler_front_end_without_gpu():
    with pytest.raises(ValueError):
        fastgl.FusedMapSampler([5], prob="p", mask="m")
    with pytest.raises(NotImplementedError):
        fastgl.FusedMapSampler([5], replace=True)
    s = fastgl.FusedMapSampler([15, 10, 5])
    with pytest.raises(RuntimeError, match="not set"):
        s.sample_blocks(None, torch.arange(4))
    b = fastgl.Block(torch.tensor([0, 2, 2, 5], dtype=torch.int32), torch.tensor([3, 1, 0, 2, 4], dtype=torch.int32), 5, 3)
    src, dst = b.edges()
    assert dst.tolist() == [0, 0, 2, 2, 2] and b.num_src_nodes() == 5 and b.num_dst_nodes() == 3 and b.num_edges() == 5
    assert b.in_degrees().tolist() == [2, 0, 3]
    assert b.int().to("cpu") is b and b.to(torch.device("cpu")) is b
    with pytest.raises(RuntimeError, match="live on the device"):
        b.to("cuda")
    b.edge_ptr.fgl_longest_row = 3
    c = b.clone()
    assert c.edge_ptr.data_ptr() != b.edge_ptr.data_ptr() and c.edge_ptr.fgl_longest_row == 3
    assert c.edges()[0].tolist() == src.tolist() and c.num_src_nodes() == 5
    for bad in (1, -2):
        with pytest.raises(ValueError):
            fastgl.FusedMapSampler([5], graph_slots=bad)
    with pytest.raises(ValueError):
        fastgl.FusedMapSampler([5], id_order="arrival", deterministic=True)
    with pytest.raises(RuntimeError, match="fused"):
        fastgl.FusedMapSampler([5], fused=False).begin_sample(torch.arange(4))
    with pytest.raises(RuntimeError, match="not set"):
        fastgl.FusedMapSampler([5]).begin_sample(torch.arange(4))


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(L, "_lib", None)
    monkeypatch.setattr(L, "LIB_PATH", "/nonexistent/libfastgl_hip.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        L.lib()


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asking for more ends with a message that says so (no GPU is touched)."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "--gpus 1" in (r.stdout + r.stderr)


def test_compiled_module_loads_and_exports_the_reference_names():
    """The torch extension module `fastgl` built from csrc/fastgl_module.cpp: loadable without a GPU, exports the ten
    operator names the reference's Python code calls (aggregate_acc.cpp:601-621), raises RuntimeError on host tensors."""
    import glob
    import importlib.util
    paths = glob.glob(os.path.join(ROOT, "fastgl-ae_amd", "fastgl_ext", "fastgl*.so"))
    assert paths, "make -C fastgl-ae_amd/csrc module"
    spec = importlib.util.spec_from_file_location("fastgl", paths[0])
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    for name in ("sample_node", "transfer_edge_id", "cal_deg", "exclusive_sum", "forward_gcn", "backward_gcn", "forwaed_gin",
                 "backward_gin", "forward_gat", "backward_gat"):
        assert callable(getattr(mod, name)), name
    assert mod.abi_version() == fastgl.lib().fgl_abi_version()
    cpu = torch.zeros(4, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        mod.sample_node(cpu, cpu, cpu, cpu, 4, 2)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        mod.transfer_edge_id(cpu, cpu, cpu, 4, 8, 4, 4)
    with pytest.raises(TypeError):
        mod.cal_deg(cpu)  # positional signature as the reference's: (edges, nodes_num)


def test_traffic_record_is_only_used_while_it_matches(tmp_path, monkeypatch, capsys):
    """bench.py reports roofline.traffic from the tracked counter summary only while the kernel source's hash and the
    bytes per launch match the run."""
    import importlib.util
    import json
    spec = importlib.util.spec_from_file_location("bench_mod", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    rec = {"workload": "c3", "source_sha16": bench.source_hash(), "algorithmic_bytes_per_launch": 800e6, "traffic_bytes_per_launch": 700e6}
    f = tmp_path / "p.md"
    f.write_text("# x\n\ntraffic_record: " + json.dumps(rec) + "\n")
    monkeypatch.setattr(bench, "TRAFFIC_PROFILE", str(f))
    assert bench.traffic_from_profile("c3", 810e6) == 700e6
    assert bench.traffic_from_profile("c3", 900e6) is None       # another problem size
    assert bench.traffic_from_profile("c2", 800e6) is None       # another workload
    rec["source_sha16"] = "0" * 16
    f.write_text("traffic_record: " + json.dumps(rec) + "\n")
    assert bench.traffic_from_profile("c3", 800e6) is None       # the kernel has changed since
    monkeypatch.setattr(bench, "TRAFFIC_PROFILE", str(tmp_path / "missing.md"))
    assert bench.traffic_from_profile("c3", 800e6) is None


def test_size_limits_are_stated_before_anything_is_launched():
    """Sizes that would overflow the library's 32-bit offsets come back as errors with the limit in the message."""
    lib = fastgl.lib()
    fake = C.c_void_p(0x1000)  # never dereferenced: every call below fails its size checks first
    # seeds x fanout beyond int32 edge offsets
    assert lib.fgl_sample_node(fake, 1, fake, 10, fake, 20_000_000, None, 192, 0, 0, fake, None, fake, None, None, None, fake, 1 << 40, None) == 1
    assert b"overflows int32" in lib.fgl_last_error()
    # a hop of the all-hops plan that could produce more than 2^31 edges
    fan = (C.c_int32 * 2)(192, 192)
    assert lib.fgl_sample_blocks_plan(1 << 30, 20_000_000, fan, 2, None, 0, None, None, None, None, None) == 1
    assert b"beyond int32" in lib.fgl_last_error()
    # hop counts and fanouts outside the supported range
    fan1 = (C.c_int32 * 1)(193)
    assert lib.fgl_sample_blocks_plan(100, 10, fan1, 1, None, 0, None, None, None, None, None) == 1
    assert b"fanout" in lib.fgl_last_error()
    fan33 = (C.c_int32 * 33)(*([2] * 33))
    assert lib.fgl_sample_blocks_plan(100, 10, fan33, 33, None, 0, None, None, None, None, None) == 1
    assert b"hops" in lib.fgl_last_error()
    # a transposed block asked for a hop that the call does not have
    fan2 = (C.c_int32 * 2)(5, 5)
    assert lib.fgl_sample_blocks_plan(100, 10, fan2, 2, None, 0b100, None, None, None, None, None) == 1
    assert b"beyond the 2" in lib.fgl_last_error()
    # an id-map call whose local ids would not fit 31 bits next to the pending marker
    assert lib.fgl_idmap_map_src(fake, 64, fake, fake, (1 << 31) - 1, None, 10, None, None, fake, 100, 0, None, fake, 1 << 40, None) == 1
    assert b"31 bits" in lib.fgl_last_error()
    # a table that is not a power of two
    assert lib.fgl_idmap_insert_dst(fake, 1000, fake, 10, None, None, None, None) == 1
    assert b"power of two" in lib.fgl_last_error()
    # more ids than a table takes at load 1/2
    assert lib.fgl_idmap_insert_dst(fake, 64, fake, 33, None, None, None, None) == 1
    assert b"load 1/2" in lib.fgl_last_error()
    # a transpose of more than 2^31 - 1 entries, and a batched one of a block that is too large for it
    assert lib.fgl_block_transpose(fake, fake, 10, None, 10, None, 1 << 31, fake, fake, None, None, 0, fake, 1 << 40, None) == 1
    assert b"int32 offsets" in lib.fgl_last_error()
    one = lambda v: (C.c_int64 * 1)(v)
    pp = (C.c_void_p * 1)(0x1000)
    assert lib.fgl_block_transpose_batch(1, pp, pp, one(10), one(10), one(1 << 20), pp, pp, None, None, fake, 1 << 40, None) == 1
    assert b"too large" in lib.fgl_last_error()
    assert lib.fgl_block_transpose_batch(9, pp, pp, one(10), one(10), one(10), pp, pp, None, None, fake, 1 << 40, None) == 1
    assert b"blocks outside" in lib.fgl_last_error()
