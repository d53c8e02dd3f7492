"""CPU-only checks: the C-ABI library loads and exports every symbol the header
declares, the snapshot codec, option handling and refusal of CPU tensors.  No
kernel is launched here."""
import ctypes
import json
import os
import re
import struct
import subprocess
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from diffcache_amd import _hip
    header = open(os.path.join(ROOT, "include", "diffcache_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(dc_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 20
    lib = ctypes.CDLL(_hip.LIB_PATH)
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert declared == set(_hip.SYMBOLS), declared ^ set(_hip.SYMBOLS)
    assert _hip.lib.dc_version() == 1


def test_layer_args_struct_matches_header_order():
    from diffcache_amd import _hip
    header = open(os.path.join(ROOT, "include", "diffcache_hip.h")).read()
    body = header[header.index("typedef struct dc_layer_args {"):header.index("} dc_layer_args;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    names = []
    for decl in body.split(";"):
        decl = decl.replace("typedef struct dc_layer_args {", "").strip()
        if not decl:
            continue
        for part in decl.split(","):
            names.append(re.findall(r"([A-Za-z_][A-Za-z0-9_]*)\s*$", part.strip())[0])
    assert names == [f[0] for f in _hip.LayerArgs._fields_]


def test_one_kernel_guard_rule():
    """When a short-context call may run as one kernel (all its blocks wait for each other, so two
    launches must never overlap): the rule of dc_one_kernel_guard, every combination."""
    from diffcache_amd import _hip
    g = _hip.lib.dc_one_kernel_guard
    auto, excl, never = _hip.ONE_KERNEL_AUTO, _hip.ONE_KERNEL_EXCLUSIVE, _hip.ONE_KERNEL_NEVER
    for capturing in (0, 1):
        for have_prev in (0, 1):
            for same in (0, 1):
                for done in (0, 1):
                    assert g(never, capturing, have_prev, same, done) == 0
                    assert g(excl, capturing, have_prev, same, done) == 1
                    want = 0 if capturing else int((not have_prev) or same or done)
                    assert g(auto, capturing, have_prev, same, done) == want, (capturing, have_prev, same, done)
    # the case the rule exists for: an earlier launch on another stream that has not finished
    assert g(auto, 0, 1, 0, 0) == 0
    # no GPU here: nothing has failed, and asking costs nothing
    assert _hip.decode_layer_errors() == 0
    assert _hip.last_route() == _hip.ROUTE_ATTEND_ONLY


def test_route_of_a_region_too_long_for_the_sketch_scan():
    """The sketch scan names a row in 22 bits; dc_decode_layer streams the bf16 keys of a longer
    region instead (same ids).  dc_decode_layer_route follows no pointers, so it runs without a GPU."""
    from diffcache_amd import _hip
    a = _hip.LayerArgs()
    a.n_b, a.n_h, a.group, a.hd, a.budget, a.n_sink = 1, 1, 4, 128, 64, 4
    a.sketch_codes = 0x1000          # only looked at for "is there a sketch"
    a.order = _hip.ORDER_BEST
    a.recent_lo = 4 + (1 << 22)
    assert _hip.lib.dc_decode_layer_route(ctypes.byref(a)) == _hip.ROUTE_SKETCH
    a.recent_lo = 4 + (1 << 22) + 1
    assert _hip.lib.dc_decode_layer_route(ctypes.byref(a)) == _hip.ROUTE_STREAM
    a.sketch_codes = None
    a.recent_lo = 5000
    assert _hip.lib.dc_decode_layer_route(ctypes.byref(a)) == _hip.ROUTE_STREAM
    a.budget = 0
    assert _hip.lib.dc_decode_layer_route(ctypes.byref(a)) == _hip.ROUTE_ATTEND_ONLY


def test_scan_kernels_do_not_spill():
    """The scan kernels sit at the edge of their register budget (four waves per SIMD): a change
    that makes the compiler spill costs them 10 us per launch without failing any parity test, and
    a lambda that the compiler declines to inline keeps the arrays it is handed in scratch memory
    (no "spill" in the report, only a scratch size: the head-dim-256 sketch scan ran at a quarter
    of its speed that way).  Compiles the file that holds them once more with the compiler's
    resource report."""
    import shutil
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc")
    src = os.path.join(ROOT, "diffcache_amd", "csrc", "fused.hip")
    res = subprocess.run([hipcc, "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "--cuda-device-only",
                          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-fno-fast-math",
                          "-Rpass-analysis=kernel-resource-usage", "-c", src, "-o", os.devnull],
                         capture_output=True, text=True, cwd=os.path.dirname(src))
    assert res.returncode == 0, res.stderr[-2000:]
    name, seen, bad = None, 0, []
    for line in res.stderr.splitlines():
        m = re.search(r"Function Name: (\S+)", line)
        if m:
            name = m.group(1)
        m = re.search(r"(VGPRs Spill|ScratchSize \[bytes/lane\]): (\d+)", line)
        if m and name and ("prune_kernel" in name or "rescore_kernel" in name):
            seen += 1
            if int(m.group(2)) > 0:
                bad.append((name, m.group(1), int(m.group(2))))
    assert seen >= 16, "the compiler's report was not understood"
    assert not bad, bad


def test_wrappers_refuse_cpu_tensors():
    from diffcache_amd import _hip
    k = torch.zeros((1, 1, 16, 128), dtype=torch.bfloat16)
    q = torch.zeros((1, 1, 128), dtype=torch.bfloat16)
    with pytest.raises(_hip.DiffCacheError, match="no CPU path"):
        _hip.score(k, q, 0, 16)
    with pytest.raises(_hip.DiffCacheError):
        _hip.score_select(k, q, 0, 16, 4)


def test_invalid_arguments_are_reported_not_launched():
    from diffcache_amd import _hip
    rc = _hip.lib.dc_score_bf16(None, None, None, None, 1, 1, 1, 128, 0, 0, 128, 1, 1, 0, None)
    assert rc == -22 and b"null pointer" in _hip.lib.dc_last_error()
    buf = (ctypes.c_char * 4096)()
    p = ctypes.addressof(buf)
    p = (p + 255) // 256 * 256
    rc = _hip.lib.dc_score_bf16(p, p, p, None, 1, 1, 1, 96, 0, 0, 96, 1, 1, 0, None)
    assert rc == -22 and b"head_dim" in _hip.lib.dc_last_error()
    rc = _hip.lib.dc_topk_select(p, 8, p, 8, 1, 8, 4, 7, 0, None, p, 1024, None)
    assert rc == -22 and b"mode" in _hip.lib.dc_last_error()
    rc = _hip.lib.dc_topk_select(p, 100000, p, 8, 1, 100000, 4, 0, 0, None, p, 16, None)
    assert rc == -12 and b"workspace" in _hip.lib.dc_last_error()


def test_invalid_arguments_of_the_sketch_and_k_check_entry_points():
    from diffcache_amd import _hip
    lib = _hip.lib
    buf = (ctypes.c_char * 8192)()
    p = (ctypes.addressof(buf) + 255) // 256 * 256
    # dc_sketch_build_bf16(k, codes, scale, resid, n_b, n_h, n_rows, hd, k strides, code strides, keep, stream)
    rc = lib.dc_sketch_build_bf16(p, None, p, p, 1, 1, 4, 128, 0, 0, 128, 0, 0, 128, 0, None)
    assert rc == -22 and b"null pointer" in lib.dc_last_error()
    rc = lib.dc_sketch_build_bf16(p, p, p, p, 1, 1, 4, 96, 0, 0, 96, 0, 0, 96, 0, None)
    assert rc == -22 and b"head_dim" in lib.dc_last_error()
    rc = lib.dc_sketch_build_bf16(p, p, p, p, 1, 1, 4, 128, 0, 0, 128, 0, 0, 120, 0, None)
    assert rc == -22 and b"code strides" in lib.dc_last_error()
    # dc_score_select_sketch_bf16: bad order, then a workspace that is too small
    args = [p, p, p, p, p, p, 8, 1, 1, 64, 128, 0, 0, 128, 0, 0, 128, 1, 8, 1]
    rc = lib.dc_score_select_sketch_bf16(*args, 9, 0, p, 4096, None, None, None)
    assert rc == -22 and b"order" in lib.dc_last_error()
    rc = lib.dc_score_select_sketch_bf16(*args, 0, 0, p, 16, None, None, None)
    assert rc == -12 and b"workspace" in lib.dc_last_error()
    assert lib.dc_sketch_select_workspace_bytes(4, 1000, 16) == lib.dc_score_select_workspace_bytes(4, 1000, 16)
    # dc_kcheck_f32: more sizes than the kernel takes, scores stride below n_sel
    seq = (ctypes.c_int * 17)(*range(10, 27))
    rc = lib.dc_kcheck_f32(p, 64, 1, 64, 128, 1, seq, 17, 0.9, p, None, None, None)
    assert rc == -22 and b"at most 16" in lib.dc_last_error()
    rc = lib.dc_kcheck_f32(p, 8, 1, 64, 128, 1, seq, 4, 0.9, p, None, None, None)
    assert rc == -22 and b"scores_unit_stride" in lib.dc_last_error()


def test_invalid_arguments_of_the_pq_search_entry_point():
    from diffcache_amd import _hip
    lib = _hip.lib
    buf = (ctypes.c_char * 8192)()
    p = (ctypes.addressof(buf) + 255) // 256 * 256
    # dc_pq_search_bf16(k, codes, lut, q, idx_out, idx_stride, n_b, n_h, n_rows, hd, m, k strides,
    #                   n_cand, topk, state_ready, workspace, workspace_bytes, ev, ev, stream)
    head = [p, p, p, p, p, 8, 1, 1, 64, 128]
    rc = lib.dc_pq_search_bf16(*head, 24, 0, 0, 128, 16, 8, 0, p, 4096, None, None, None)
    assert rc == -22 and b"subspaces" in lib.dc_last_error()
    rc = lib.dc_pq_search_bf16(*head, 32, 0, 0, 128, 8, 16, 0, p, 4096, None, None, None)
    assert rc == -22 and b"topk <= n_cand" in lib.dc_last_error()
    rc = lib.dc_pq_search_bf16(*head, 32, 0, 0, 128, 16, 8, 0, p, 16, None, None, None)
    assert rc == -12 and b"workspace" in lib.dc_last_error()
    rc = lib.dc_pq_search_bf16(p, None, p, p, p, 8, 1, 1, 64, 128, 32, 0, 0, 128, 16, 8, 0, p, 4096, None,
                               None, None)
    assert rc == -22 and b"null pointer" in lib.dc_last_error()
    # nothing to do: no rows, or no results wanted
    assert lib.dc_pq_search_bf16(p, p, p, p, p, 8, 1, 1, 0, 128, 32, 0, 0, 128, 16, 8, 0, None, 0, None,
                                 None, None) == 0
    assert lib.dc_pq_search_workspace_bytes(8, 1000, 64) > lib.dc_score_select_workspace_bytes(8, 1000, 64)


def test_c_data_layer_handle_bookkeeping_and_errors():
    """dc_data_layer_*: the host-side mirror of lib.rs:189-404 as a C handle; everything that
    needs no GPU (creation, sizes, argument checks)."""
    from diffcache_amd import _hip
    lib = _hip.lib
    h = ctypes.c_void_p()
    assert lib.dc_data_layer_create(ctypes.byref(h), 2, 4, 96, 1000, 1, 1) == -22
    assert b"head_dim" in lib.dc_last_error() and not h.value
    assert lib.dc_data_layer_create(ctypes.byref(h), 2, 4, 128, 1000, 7, 1) == -22
    assert b"mode" in lib.dc_last_error()
    assert lib.dc_data_layer_create(ctypes.byref(h), 2, 4, 128, 1000, 1, 1) == 0 and h.value
    assert lib.dc_data_layer_ctx_len(h) == 0
    sizes = [ctypes.c_size_t() for _ in range(5)]
    assert lib.dc_data_layer_sizes(h, 64, *[ctypes.byref(x) for x in sizes]) == 0
    store, codes, scale, idx, ws = [x.value for x in sizes]
    assert store == 2 * 4 * 1000 * 128 * 2 and codes == 2 * 4 * 1000 * 128
    assert scale == 2 * 4 * 128 * 4 and idx == 2 * 4 * 64 * 4
    assert ws == lib.dc_sketch_select_workspace_bytes(8, 1000, 64)
    buf = (ctypes.c_char * 8192)()
    p = (ctypes.addressof(buf) + 255) // 256 * 256
    # not bound yet
    assert lib.dc_data_layer_prefill(h, p, p, 10, None) == -22 and b"bound" in lib.dc_last_error()
    assert lib.dc_data_layer_insert(h, p, p, None) == -22
    assert lib.dc_data_layer_query(h, p, p, 8, p, 8, None, None) == -22
    # binding: missing sketch buffers, small workspace
    assert lib.dc_data_layer_bind(h, p, p, None, None, None, p, p, ws, 64) == -22
    assert b"sketch buffers" in lib.dc_last_error()
    assert lib.dc_data_layer_bind(h, p, p, p, p, p, p, p, 16, 64) == -12
    lib.dc_data_layer_destroy(h)
    lib.dc_data_layer_destroy(None)
    assert lib.dc_data_layer_ctx_len(None) == -1


def test_data_layer_option_errors():
    from diffcache_amd import DiffCacheHIP
    from diffcache_amd._hip import DiffCacheError
    with pytest.raises(ValueError, match="Unknown option"):      # lib.rs:579
        DiffCacheHIP(1, 8, 2, 128, bogus=1)
    with pytest.raises(AssertionError, match="multiple"):        # lib.rs:294
        DiffCacheHIP(1, 7, 2, 128)
    with pytest.raises(DiffCacheError, match="no CPU path"):
        DiffCacheHIP(1, 8, 2, 128, device="cpu", max_ctx_len=8)


def test_bench_refuses_more_than_one_gpu():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                         capture_output=True, text=True)
    assert res.returncode != 0 and "one GPU" in res.stderr


def test_bench_refuses_an_unknown_shape_key():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--shape", "batch=2,rows=5"],
                         capture_output=True, text=True)
    assert res.returncode != 0 and "bad --shape" in res.stderr


# ---------------------------------------------------------------- snapshot codec

def test_varint_known_answers():
    from diffcache_amd import snapshot
    assert snapshot._varint(0) == b"\x00"
    assert snapshot._varint(250) == b"\xfa"
    assert snapshot._varint(251) == b"\xfb\xfb\x00"
    assert snapshot._varint(65535) == b"\xfb\xff\xff"
    assert snapshot._varint(65536) == b"\xfc\x00\x00\x01\x00"
    assert snapshot._varint(1 << 32) == b"\xfd" + struct.pack("<Q", 1 << 32)


def test_snapshot_bytes_of_a_tiny_index(tmp_path):
    """Hand-assembled bincode of a 2-node, dim-2 index (field order of
    nsw.rs:64-72, options of nsw.rs:22-31)."""
    from diffcache_amd import snapshot
    path = str(tmp_path / "t.idx")
    keys = np.float32([[1.0, 2.0], [3.0, 4.0]])
    vals = np.float32([[5.0, 6.0], [7.0, 8.0]])
    snapshot.write(path, keys, vals, m=16, ef_cons=200, n_max=1000, r_sq=4.0, name="l0",
                   attn_mass_threshold=0.5, k_check_seq=[100, 300])
    want = (b"\x02" + b"\x00\x00" + b"\x01\x00"                       # 2 nodes: (id, 0 edges)
            + b"\x04" + keys.tobytes() + b"\x04" + vals.tobytes()     # Vec<f32> x 2
            + b"\x10" + b"\xc8" + b"\xfb\xe8\x03"                     # m 16, ef_cons 200, n_max 1000
            + struct.pack("<f", 4.0) + b"\x02l0" + struct.pack("<f", 0.5)
            + b"\x02" + b"\x64" + b"\xfb\x2c\x01"                     # k_check_seq [100, 300]
            + b"\x02" + b"\x02")                                      # dim, num_nodes
    assert open(path, "rb").read() == want
    snap = snapshot.read(path)
    assert np.array_equal(snap["keys"], keys) and np.array_equal(snap["vals"], vals)
    assert snap["options"]["k_check_seq"] == [100, 300] and snap["options"]["name"] == "l0"
    assert snap["dim"] == 2 and snap["num_nodes"] == 2


def test_snapshot_with_edges_as_the_reference_writes_them(tmp_path):
    """A file whose nodes carry edge lists (what the reference saves) must load."""
    from diffcache_amd import snapshot
    keys = np.float32([[1.0], [2.0], [3.0]])
    raw = (b"\x03" + b"\x00\x02\x01\x02" + b"\x01\x01\x00" + b"\x02\x00"
           + b"\x03" + keys.tobytes() + b"\x03" + keys.tobytes()
           + b"\x10\xc8\x0a" + struct.pack("<f", 4.0) + b"\x01x" + struct.pack("<f", 0.9) + b"\x00"
           + b"\x01\x03")
    path = str(tmp_path / "e.idx")
    open(path, "wb").write(raw)
    snap = snapshot.read(path, keep_edges=True)
    assert snap["edges"] == [[1, 2], [0], []]
    assert np.array_equal(snap["keys"], keys)


def test_snapshot_roundtrip_many_nodes(tmp_path):
    from diffcache_amd import snapshot
    rng = np.random.default_rng(0)
    n, dim = 70000, 8                      # crosses the 251 and 65536 varint boundaries
    keys = rng.standard_normal((n, dim)).astype(np.float32)
    vals = rng.standard_normal((n, dim)).astype(np.float32)
    path = str(tmp_path / "big.idx")
    snapshot.write(path, keys, vals, m=16, ef_cons=200, n_max=n, r_sq=1.5, name="l003b001h002",
                   attn_mass_threshold=0.9, k_check_seq=[1048576])
    snap = snapshot.read(path)
    assert np.array_equal(snap["keys"], keys) and np.array_equal(snap["vals"], vals)
    assert snap["num_nodes"] == n and snap["options"]["n_max"] == n
