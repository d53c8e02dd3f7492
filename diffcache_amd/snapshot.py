"""Reader/writer for the reference's per-unit index snapshot files.

Layout (diffcache_cpu/src/nsw.rs:58-72 ``IndexSnapshot``, written with bincode 2
``config::standard()`` at nsw.rs:779-794): little endian; every integer is a
varint (< 251: one byte; 251 + u16; 252 + u32; 253 + u64); ``f32`` is four raw
bytes; ``Vec`` and ``String`` carry a varint length first.  Field order::

    nodes:   Vec<{id: u32, edges: Vec<u32>}>
    keys:    Vec<f32>        num_nodes * dim, row major (bf16 widened on save)
    vals:    Vec<f32>
    options: {m, ef_cons, n_max: usize, r_sq: f32, name: String,
              attn_mass_threshold: f32, k_check_seq: Vec<usize>}
    dim:       usize
    num_nodes: usize

The HBM store keeps no graph, so files written here carry empty edge lists;
files written by the reference are read with their edges skipped.
"""
from __future__ import annotations

import struct
from typing import Dict, List, Sequence

import numpy as np


def _varint(u: int) -> bytes:
    if u < 251:
        return bytes([u])
    if u < 1 << 16:
        return b"\xfb" + struct.pack("<H", u)
    if u < 1 << 32:
        return b"\xfc" + struct.pack("<I", u)
    return b"\xfd" + struct.pack("<Q", u)


def _nodes_without_edges(n: int) -> bytes:
    """Vec<NodeSnapshot> for ids 0..n-1, each with an empty edge list, built
    with numpy (one id varint + one zero length byte per node)."""
    out = [_varint(n)]
    a = min(n, 251)
    if a:
        small = np.zeros((a, 2), np.uint8)
        small[:, 0] = np.arange(a, dtype=np.uint8)
        out.append(small.tobytes())
    b = min(n, 1 << 16)
    if b > 251:
        ids = np.arange(251, b, dtype="<u2")
        mid = np.zeros((len(ids), 4), np.uint8)
        mid[:, 0] = 251
        mid[:, 1:3] = ids.view(np.uint8).reshape(-1, 2)
        out.append(mid.tobytes())
    if n > 1 << 16:
        ids = np.arange(1 << 16, n, dtype="<u4")
        big = np.zeros((len(ids), 6), np.uint8)
        big[:, 0] = 252
        big[:, 1:5] = ids.view(np.uint8).reshape(-1, 4)
        out.append(big.tobytes())
    return b"".join(out)


def write(path: str, keys_f32: np.ndarray, vals_f32: np.ndarray, *, m: int, ef_cons: int, n_max: int,
          r_sq: float, name: str, attn_mass_threshold: float, k_check_seq: Sequence[int]) -> None:
    keys = np.ascontiguousarray(keys_f32, dtype="<f4")
    vals = np.ascontiguousarray(vals_f32, dtype="<f4")
    n, dim = keys.shape
    if vals.shape != (n, dim):
        raise AssertionError("keys and vals must have the same shape")
    name_b = name.encode("utf-8")
    with open(path, "wb") as f:
        f.write(_nodes_without_edges(n))
        f.write(_varint(n * dim))
        f.write(keys.tobytes())
        f.write(_varint(n * dim))
        f.write(vals.tobytes())
        f.write(_varint(m) + _varint(ef_cons) + _varint(n_max))
        f.write(struct.pack("<f", r_sq))
        f.write(_varint(len(name_b)) + name_b)
        f.write(struct.pack("<f", attn_mass_threshold))
        f.write(_varint(len(k_check_seq)) + b"".join(_varint(int(x)) for x in k_check_seq))
        f.write(_varint(dim) + _varint(n))


class _Reader:
    def __init__(self, buf: bytes) -> None:
        self.b = memoryview(buf)
        self.p = 0

    def varint(self) -> int:
        t = self.b[self.p]
        self.p += 1
        if t < 251:
            return t
        size = {251: 2, 252: 4, 253: 8, 254: 16}.get(t)
        if size is None:
            raise ValueError(f"bad varint tag {t} at byte {self.p - 1}")
        v = int.from_bytes(self.b[self.p:self.p + size], "little")
        self.p += size
        return v

    def f32(self) -> float:
        v = struct.unpack_from("<f", self.b, self.p)[0]
        self.p += 4
        return v

    def f32_vec(self) -> np.ndarray:
        n = self.varint()
        a = np.frombuffer(self.b, dtype="<f4", count=n, offset=self.p).copy()
        self.p += 4 * n
        return a

    def string(self) -> str:
        n = self.varint()
        s = bytes(self.b[self.p:self.p + n]).decode("utf-8")
        self.p += n
        return s


def read(path: str, keep_edges: bool = False) -> Dict:
    with open(path, "rb") as f:
        r = _Reader(f.read())
    n_nodes = r.varint()
    edges: List[List[int]] = []
    for i in range(n_nodes):
        node_id = r.varint()
        if node_id != i:
            raise ValueError(f"snapshot node {i} carries id {node_id}")
        deg = r.varint()
        e = [r.varint() for _ in range(deg)]
        if keep_edges:
            edges.append(e)
    keys = r.f32_vec()
    vals = r.f32_vec()
    options = {"m": r.varint(), "ef_cons": r.varint(), "n_max": r.varint(), "r_sq": r.f32(),
               "name": r.string(), "attn_mass_threshold": r.f32()}
    options["k_check_seq"] = [r.varint() for _ in range(r.varint())]
    dim = r.varint()
    num_nodes = r.varint()
    if r.p != len(r.b):
        raise ValueError("trailing bytes in snapshot")
    if len(keys) != n_nodes * dim or len(vals) != n_nodes * dim:
        raise ValueError("snapshot key/value length does not match nodes * dim")
    out = {"keys": keys.reshape(n_nodes, dim), "vals": vals.reshape(n_nodes, dim), "options": options,
           "dim": dim, "num_nodes": num_nodes, "n_nodes_stored": n_nodes}
    if keep_edges:
        out["edges"] = edges
    return out
