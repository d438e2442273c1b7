"""Host-side checks that need no GPU: the C-ABI library loads and exports every symbol
the header declares, argument validation works, and the weight packing of the colour
network reproduces the oracle when replayed through a numpy model of the matrix-core
data flow (32x32 accumulator layout: lane l -> column l%32, register v -> row
8*(v/4) + 4*(l/32) + v%4)."""
import ctypes as C
import os
import re

import numpy as np
import pytest
import torch

from landmark_amd import _lib as L
from landmark_amd import scenes
from oracle import gridnerf_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(L.SO_PATH):
        from landmark_amd import build

        build.build(verbose=False)
    return L.load()


def test_every_declared_symbol_is_exported(lib):
    header = open(os.path.join(ROOT, "include", "landmark_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(lm_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations found"
    assert declared == set(L.SYMBOLS), f"binding table and header differ: {declared ^ set(L.SYMBOLS)}"
    for name in declared:
        assert hasattr(lib, name), name


def test_struct_sizes_match_header_layout():
    assert C.sizeof(L.LmPlane) == 48
    assert C.sizeof(L.LmGeom) == 152  # 40 B scalars, 2 pointers, inv_aabb + pad, pointer, 4 ints, 7 floats, 2 ints, 2 floats, pointer
    assert C.sizeof(L.LmModel) % 8 == 0


def test_header_compiles_as_c_and_matches_the_binding_field_by_field(tmp_path):
    """The header is plain C (gcc -std=c11 -pedantic), and every field of its three structs sits at the offset and
    has the size the ctypes mirror gives it: a C caller and the Python binding see the same memory."""
    import shutil
    import subprocess

    cc = shutil.which("gcc") or shutil.which("cc")
    if cc is None:
        pytest.skip("no C compiler")
    pairs = [("lm_plane", L.LmPlane), ("lm_geom", L.LmGeom), ("lm_model", L.LmModel)]
    lines = ['#include "landmark_hip.h"', "#include <stddef.h>", "#include <stdio.h>", "int main(void) {"]
    for cname, st in pairs:
        lines.append(f'  printf("{cname} . %zu %zu\\n", (size_t)0, sizeof({cname}));')
        for field, _ in st._fields_:
            lines.append(f'  printf("{cname} {field} %zu %zu\\n", offsetof({cname}, {field}), sizeof((({cname} *)0)->{field}));')
    lines += ['  printf("const LM_ABI_VERSION %d 0\\n", LM_ABI_VERSION);', '  printf("const LM_STAT_WORDS %d 0\\n", LM_STAT_WORDS);',
              '  printf("const LM_STAT_OVERFLOW %d 0\\n", LM_STAT_OVERFLOW);', '  printf("const LM_MAX_PLANES %d 0\\n", LM_MAX_PLANES);',
              '  printf("const LM_STATIC_WORKSPACE_BYTES %u 0\\n", (unsigned)LM_STATIC_WORKSPACE_BYTES);', "  return 0;", "}"]
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines) + "\n")
    exe = tmp_path / "layout"
    subprocess.check_call([cc, "-std=c11", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(ROOT, "include"),
                           str(src), "-o", str(exe)])
    seen = {}
    for row in subprocess.check_output([str(exe)], text=True).splitlines():
        a, b, off, size = row.split()
        seen[(a, b)] = (int(off), int(size))
    for cname, st in pairs:
        assert seen[(cname, ".")][1] == C.sizeof(st), cname
        for field, _ in st._fields_:
            d = getattr(st, field)
            assert seen[(cname, field)] == (d.offset, d.size), (cname, field)
    assert seen[("const", "LM_ABI_VERSION")][0] == L.LM_ABI_VERSION
    assert seen[("const", "LM_STAT_WORDS")][0] == L.LM_STAT_WORDS
    assert seen[("const", "LM_STAT_OVERFLOW")][0] == L.LM_STAT_OVERFLOW
    assert seen[("const", "LM_MAX_PLANES")][0] == L.LM_MAX_PLANES
    assert seen[("const", "LM_STATIC_WORKSPACE_BYTES")][0] == L.LM_STATIC_WORKSPACE_BYTES


def test_argument_validation_returns_status_not_abort(lib):
    g = L.LmGeom()
    g.S = 0
    rc = lib.lm_sample_cull(C.byref(g), None, 4, None, None, None, None, None, None, None)
    assert rc == -1 and b"S must be positive" in lib.lm_last_error()
    assert lib.lm_mlp_packed_bytes(7, 144) == 0
    assert lib.lm_mlp_packed_bytes(L.LM_MLP_F32, 100) == 0  # K not a multiple of 16
    pl = (L.LmPlane * 1)()
    rc = lib.lm_gather_density_xyz(pl, 1, None, None, 10, None, None)
    assert rc == -1 and b"null table" in lib.lm_last_error()
    assert lib.lm_gather_density_xyz(pl, 13, None, None, 10, None, None) == -1
    assert lib.lm_relayout_nchw_to_hwc(None, None, 4, 4, 4, 0, None) == -1
    # a table row must stay below 2^31 elements: the kernels step between corners with 32-bit offsets
    pl[0].plane = pl[0].line = 16
    pl[0].H, pl[0].W, pl[0].Len, pl[0].C = 4, 1 << 26, 4, 32
    rc = lib.lm_gather_density_xyz(pl, 1, None, None, 10, None, None)
    assert rc == -1 and b"2^31" in lib.lm_last_error()


def test_coarse_occupancy_sizes_and_validation(lib):
    """Two tables of one byte per block of 8 x 8 x 8 cells (the coarse level and the undilated one it is built from);
    null buffers and empty volumes are refused before anything is launched."""
    assert lib.lm_occupancy_coarse_bytes(256, 256, 256) == 2 * 33 ** 3
    assert lib.lm_occupancy_coarse_bytes(7, 8, 64) == 2 * 1 * 2 * 9
    assert lib.lm_occupancy_coarse_bytes(0, 8, 8) == 0
    assert lib.lm_pack_occupancy_coarse(None, 8, 8, 8, None, None) == -1 and b"null" in lib.lm_last_error()
    assert lib.lm_pack_occupancy_coarse(16, 0, 8, 8, 16, None) == -1 and b"empty" in lib.lm_last_error()


def _host_model(S=128, C=48, n=3):
    """An lm_model good enough for size queries (pointers are never dereferenced on the host)."""
    m = L.LmModel()
    m.geom.S, m.geom.sampler = S, L.LM_SAMPLER_HULL
    m.geom.tab_a = m.geom.tab_t = 16
    m.n_planes = n
    for k in range(n):
        for arr, c in ((m.density, 16), (m.app, C)):
            arr[k].plane = arr[k].line = 16
            arr[k].H = arr[k].W = arr[k].Len = 8
            arr[k].C = c
    m.mlp_prec = L.LM_MLP_F16X2
    return m


def test_workspace_size_grows_with_chunk(lib):
    m = _host_model()
    a = lib.lm_render_workspace_bytes(C.byref(m), 1024)
    b = lib.lm_render_workspace_bytes(C.byref(m), 2048)
    assert 0 < a < b
    assert lib.lm_render_workspace_bytes(C.byref(m), 0) == 0
    # channel counts the fused appearance kernel does not cover need the product matrix as well
    c = lib.lm_render_workspace_bytes(C.byref(_host_model(C=12, n=4)), 2048)
    assert c > b


# ---------------------------------------------------------------- packing replay
def row_of(v, h):
    return 8 * (v // 4) + 4 * h + v % 4


def _layout(prec, K):
    E = (4 if prec == L.LM_MLP_F32 else 2) * (2 if prec == L.LM_MLP_F16X2 else 1)
    al = lambda x: (x + 255) & ~255
    o = 0
    out = {}
    for name, n in (("basis", 32 * K * E), ("w1", 4 * 80 * 64 * E), ("b1", 512), ("w2", 4 * 64 * 64 * E), ("b2", 512), ("w3", 64 * 64 * E), ("b3", 128)):
        out[name] = o
        o = al(o + n)
    out["total"] = o
    return out


def _frags(buf, off, n_blocks, n_slots, G, dt, parts=1):
    steps = n_slots // G
    n = n_blocks * steps * parts * 64 * G
    a = np.frombuffer(buf, dtype=dt, count=n, offset=off).astype(np.float64)
    return a.reshape(n_blocks, steps, parts, 64, G).sum(axis=2)  # hi + lo


def _mma_layer(A, slots):
    """A: [nb, steps, 64, G] fragments; slots: [n_samples, 2(h), n_slots] -> D [n_samples, nb, 32 rows]"""
    nb, steps, _, G = A.shape
    Ar = A.reshape(nb, steps, 2, 32, G)  # lane = h*32 + i
    sl = slots.reshape(slots.shape[0], 2, steps, G)
    return np.einsum("bthig,nhtg->nbi", Ar.astype(np.float64), sl.astype(np.float64))


def _regs(D):
    """D [n, nb, 32] -> per-lane-half registers [n, 2, nb*16] (v = 0..15 per block)"""
    n, nb, _ = D.shape
    out = np.zeros((n, 2, nb, 16))
    for h in range(2):
        for v in range(16):
            out[:, h, :, v] = D[:, :, row_of(v, h)]
    return out.reshape(n, 2, nb * 16)


@pytest.mark.parametrize("prec,dt,tol", [(L.LM_MLP_F32, np.float32, 2e-6), (L.LM_MLP_F16, np.float16, 3e-3), (L.LM_MLP_F16X2, np.float16, 2e-6)])
def test_packed_weights_replay_matches_oracle(lib, prec, dt, tol):
    p = scenes.make_params(seed=11, gridSize=(4, 4, 4), density_n_comp=4, app_n_comp=16, ndims=3, resMode=(1,))
    K = 48
    n = lib.lm_mlp_packed_bytes(prec, K)
    lay = _layout(prec, K)
    assert n == lay["total"]
    host = np.zeros(n, np.uint8)
    arrs = [np.ascontiguousarray(t.numpy()) for t in (p.basis_mat, p.mlp_w[0], p.mlp_b[0], p.mlp_w[1], p.mlp_b[1], p.mlp_w[2], p.mlp_b[2])]
    rc = lib.lm_mlp_pack(prec, K, *[a.ctypes.data for a in arrs], host.ctypes.data)
    assert rc == 0
    buf = host.tobytes()
    G = 1 if prec == L.LM_MLP_F32 else 8
    CW = 4 if prec == L.LM_MLP_F32 else 8
    parts = 2 if prec == L.LM_MLP_F16X2 else 1
    _f = _frags
    globals()["_frags"] = lambda *a: _f(*a, parts=parts)
    g = torch.Generator().manual_seed(1)
    ns = 37
    prod = torch.randn(ns, K, generator=g)
    view = torch.randn(ns, 3, generator=g)
    # basis: lane-half h reads channels 2W*(s/W) + W*h + s%W
    ch = np.array([[2 * CW * (s // CW) + CW * h + s % CW for s in range(K // 2)] for h in range(2)])
    slots = prod.numpy()[:, ch]  # [n, 2, K/2]
    feat_rows = _mma_layer(_frags(buf, lay["basis"], 1, K // 2, G, dt), slots)  # [n,1,32]
    ref_feat = O.F.linear(prod, p.basis_mat).numpy()
    assert np.allclose(feat_rows[:, 0, :27], ref_feat, atol=tol * 10)
    assert np.all(feat_rows[:, 0, 27:] == 0)
    raw = _regs(feat_rows)  # [n,2,16]
    raw[:, 1, 12:15] = view.numpy()
    raw[:, :, 15] = 0
    s1 = np.concatenate([raw, np.sin(raw), np.cos(raw), np.sin(2 * raw), np.cos(2 * raw)], axis=2)  # [n,2,80]
    bias = lambda name, nb: np.frombuffer(buf, np.float32, nb * 32, lay[name]).reshape(nb, 2, 16)
    h1 = np.maximum(_regs(_mma_layer(_frags(buf, lay["w1"], 4, 80, G, dt), s1)) + bias("b1", 4).transpose(1, 0, 2).reshape(2, 64), 0)
    h2 = np.maximum(_regs(_mma_layer(_frags(buf, lay["w2"], 4, 64, G, dt), h1)) + bias("b2", 4).transpose(1, 0, 2).reshape(2, 64), 0)
    o = _regs(_mma_layer(_frags(buf, lay["w3"], 1, 64, G, dt), h2)) + bias("b3", 1).transpose(1, 0, 2).reshape(2, 16)
    globals()["_frags"] = _f
    rgb = 1 / (1 + np.exp(-o[:, 0, :3]))
    ref = O.mlp_render(p, view, torch.from_numpy(ref_feat)).numpy()
    assert np.allclose(rgb, ref, atol=tol)
