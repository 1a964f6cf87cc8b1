"""Host-side checks that need no GPU: the C-ABI library loads, exports every symbol include/vetrast.h declares, and its
pure-host functions (layer sizes, workspace layout, status strings, argument validation) behave."""
import ctypes as C
import os
import re

import pytest

from vet_amd import abi, synthetic
from vet_amd.rasterizer import fill_forward_args, make_params, make_views

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "vetrast.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(vetrast_[a-z_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = abi.load_library()
    names = declared_functions()
    assert len(names) >= 18
    assert sorted(abi.SYMBOLS) == names, "vet_amd/abi.py and include/vetrast.h disagree"
    for n in names:
        assert getattr(lib, n) is not None


def test_struct_sizes_are_the_c_ones():
    # sizes the C compiler gives the structs of include/vetrast.h (LP64)
    assert C.sizeof(abi.View) == 5 * 4 + 9 * 4
    assert C.sizeof(abi.Params) == 21 * 4 + abi.MAX_LAYERS * 4 + 2 * 4
    assert C.sizeof(abi.LiftArgs) == 8 + 4 * 8 + 2 * 4 + 2 * 8 + C.sizeof(abi.View) + 8 + 4 * 4 + 2 * 8 == 160
    assert abi.LiftArgs.loss_image.offset % 8 == 0
    assert C.sizeof(abi.ForwardArgs) % 8 == 0
    assert abi.BackwardArgs.grad_out.offset == C.sizeof(abi.ForwardArgs)


def test_every_struct_field_sits_where_the_c_compiler_puts_it(tmp_path):
    """Compiles include/vetrast.h with gcc and compares size and every field offset of every struct with the ctypes
    mirror in vet_amd/abi.py (field names are the same on both sides)."""
    import subprocess

    pairs = [("vetrast_view", abi.View), ("vetrast_params", abi.Params), ("vetrast_workspace_layout", abi.WorkspaceLayout),
             ("vetrast_forward_args", abi.ForwardArgs), ("vetrast_backward_args", abi.BackwardArgs),
             ("vetrast_adam_args", abi.AdamArgs), ("vetrast_lift_args", abi.LiftArgs), ("vetrast_pack_args", abi.PackArgs)]
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "vetrast.h"', 'int main(void) {']
    for cname, mirror in pairs:
        lines.append(f'printf("{cname} size %zu\\n", sizeof({cname}));')
        for field, _ in mirror._fields_:
            lines.append(f'printf("{cname} {field} %zu\\n", offsetof({cname}, {field}));')
    lines += ['return 0; }']
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c99", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    got = {}
    for line in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines():
        cname, field, value = line.split()
        got[(cname, field)] = int(value)
    for cname, mirror in pairs:
        assert got[(cname, "size")] == C.sizeof(mirror), cname
        for field, _ in mirror._fields_:
            assert got[(cname, field)] == getattr(mirror, field).offset, (cname, field)
        # the sizes agree and the last mirrored field ends inside the struct: no member of the C struct is missing
        last, last_type = mirror._fields_[-1]
        assert getattr(mirror, last).offset + C.sizeof(last_type) <= C.sizeof(mirror)


def test_layer_sizes_halve_with_integer_division():
    lib = abi.load_library()
    w = (C.c_int32 * 5)()
    h = (C.c_int32 * 5)()
    assert lib.vetrast_layer_sizes(1920, 1080, 4, w, h) == 0
    assert list(w)[:4] == [1920, 960, 480, 240] and list(h)[:4] == [1080, 540, 270, 135]
    assert lib.vetrast_layer_sizes(25, 13, 3, w, h) == 0
    assert list(w)[:3] == [25, 12, 6] and list(h)[:3] == [13, 6, 3]
    assert lib.vetrast_layer_sizes(25, 13, 6, w, h) == abi.ERR_INVALID_ARG
    assert lib.vetrast_layer_sizes(0, 13, 1, w, h) == abi.ERR_INVALID_ARG


def test_workspace_layout_is_aligned_and_disjoint():
    lib = abi.load_library()
    lay = abi.WorkspaceLayout()
    N, B, L, w, h = 2_000_000, 2, 4, 1920, 1080
    assert lib.vetrast_workspace_layout_for(N, B, L, w, h, C.byref(lay)) == 0
    # pixels are numbered tile by tile (16x16), overhanging tiles included
    tiles = [((1920 >> l) + 15) // 16 * (((1080 >> l) + 15) // 16) for l in range(L)]
    T = sum(tiles)
    P = 256 * T
    assert lay.layer_tile_base[L] == T and lay.layer_pixel_base[L] == P and lay.fragment_capacity == N * L
    assert [lay.layer_tiles_x[l] for l in range(L)] == [120, 60, 30, 15]
    assert [lay.layer_tile_base[l] for l in range(L)] == [0, tiles[0], tiles[0] + tiles[1], sum(tiles[:3])]
    # the overflow log: 256 segments, each with room for every hit of ceil(workgroups / 256) workgroups of 256 points
    groups = (N + 255) // 256
    log_records = 256 * ((groups + 255) // 256 * 256 * L)
    regions = [
        ("flags", lay.flags_base, 16),
        ("offsets", lay.offsets_base, lay.offsets_stride * B),
        ("tile_counts", lay.bin_counts_base, lay.bin_counts_stride * B),
        ("binned", lay.binned_base, N * L * 8),  # 8-byte records: one hit per layer, N <= 2^24
        ("cut_flags", lay.cut_flags_base, lay.cut_flags_stride * B),
        ("kept", lay.kept_base, lay.kept_stride * B),
        ("fragments", lay.fragments_base, lay.fragments_stride * B),
        ("transmittance", lay.transmittance_base, lay.transmittance_stride * B),
        ("weight", lay.weight_base, lay.weight_stride * B),
        ("packed", lay.packed_base, N * 32),
        ("log_cursor", lay.log_cursor_base, B * 256 * 64),
        # rooms of 1024 records where at most 512 are expected per bin (layer 0: 2 M points over 8100 tiles), 2048 elsewhere
        ("primary", lay.primary_base, (tiles[0] * 1024 + (tiles[1] + 4 * tiles[2] + 16 * tiles[3]) * 2048) * 8),
        ("views", lay.views_base, B * 160),
    ]
    # the scratch of the backward call lies on top of the overflow log, which only lives inside a forward call
    forward_tail = [("log", lay.log_base, log_records * 16), ("slots", lay.slots_base, log_records * 4)]
    backward_tail = [("partial", lay.partial_base, N * L * 32),
                     ("background_partial", lay.background_partial_base, (P + 255) // 256 * 32),
                     ("camera_partial", lay.camera_partial_base, (N + 255) // 256 * 160)]
    head_end = max(b + sz for _, b, sz in regions)
    for tail in (forward_tail, backward_tail):
        assert min(b for _, b, _ in tail) >= head_end
        srt = sorted(tail, key=lambda r: r[1])
        for (n0, b0, s0), (n1, b1, _) in zip(srt, srt[1:]):
            assert b0 + s0 <= b1, (n0, n1)
        for name, base, size in tail:
            assert base % 256 == 0 and base + size <= lay.total_bytes, name
    assert lay.log_base == lay.partial_base
    assert max(b + sz for _, b, sz in forward_tail) <= lay.forward_only_bytes
    assert lay.offsets_stride >= (P + 1) * 4 and lay.fragments_stride >= N * L * 8
    # 2 M points over 1080p: tiles at the two fine layers, 16x4 strips and single tile rows at the coarse ones
    assert lay.num_bins == tiles[0] + tiles[1] + 4 * tiles[2] + 16 * tiles[3]
    assert lay.bin_counts_stride >= (lay.num_bins + 1) * 4
    for name, base, size in regions:
        assert base % 256 == 0, name
        assert base + size <= lay.total_bytes, name
    ordered = sorted(regions, key=lambda r: r[1])
    for (n0, b0, s0), (n1, b1, _) in zip(ordered, ordered[1:]):
        assert b0 + s0 <= b1, (n0, n1)
    assert lay.partial_base < lay.forward_only_bytes <= lay.total_bytes
    assert lay.total_bytes < 0.8e9 * B  # the diet: under 0.8 GB per view at 2 M points / 1080p / 4 layers
    # the log cursors sit right behind the bin counters (one zero-fill covers both); BILINEAR_BLEND adds `projected`
    assert lay.log_cursor_base == lay.bin_counts_base + lay.bin_counts_stride * B
    assert lay.projected_stride == 0
    lay3 = abi.WorkspaceLayout()
    assert lib.vetrast_workspace_layout_for_mode(N, B, L, w, h, abi.RENDER_BILINEAR_BLEND, C.byref(lay3)) == 0
    assert lay3.projected_stride >= N * 8 and lay3.projected_base + lay3.projected_stride * B <= lay3.forward_only_bytes
    assert lib.vetrast_forward_workspace_bytes(N, B, L, w, h) == lay.total_bytes
    # invalid dimensions
    assert lib.vetrast_workspace_layout_for(N, 0, L, w, h, C.byref(lay)) == abi.ERR_INVALID_ARG
    assert lib.vetrast_workspace_layout_for(N, B, 6, w, h, C.byref(lay)) == abi.ERR_INVALID_ARG
    assert lib.vetrast_workspace_layout_for(N, B, 5, 8, 8, C.byref(lay)) == abi.ERR_INVALID_ARG  # coarsest layer empty
    assert lib.vetrast_workspace_layout_for(2_000_000_000, B, 4, w, h, C.byref(lay)) == abi.ERR_INVALID_ARG
    assert lib.vetrast_forward_workspace_bytes(N, 0, L, w, h) == 0
    # BILINEAR_BLEND: four fragments per point and layer
    full = lay.total_bytes
    assert lib.vetrast_workspace_layout_for_mode(N, B, L, w, h, abi.RENDER_BILINEAR_BLEND, C.byref(lay)) == 0
    assert lay.hits_per_layer == 4 and lay.fragment_capacity == 4 * N * L and lay.total_bytes > 3 * full
    # FUZZY_BLEND uses the FULL_BLEND lists; other mode numbers are refused
    assert lib.vetrast_workspace_layout_for_mode(N, B, L, w, h, abi.RENDER_FUZZY_BLEND, C.byref(lay)) == 0
    assert lay.hits_per_layer == 1 and lay.total_bytes == full
    assert lib.vetrast_workspace_layout_for_mode(N, B, L, w, h, 4, C.byref(lay)) == abi.ERR_UNSUPPORTED


def test_status_and_scope_names():
    lib = abi.load_library()
    assert lib.vetrast_status_string(0) == b"ok"
    for st in (abi.ERR_INVALID_ARG, abi.ERR_WORKSPACE_SMALL, abi.ERR_HIP, abi.ERR_UNSUPPORTED, abi.ERR_BAD_INPUT_DATA):
        assert lib.vetrast_status_string(st) not in (b"ok", b"unknown status")
    assert lib.vetrast_status_string(-99) == b"unknown status"
    names = [lib.vetrast_scope_name(i).decode() for i in range(abi.SCOPE_COUNT)]
    # the reference's CudaTimerSystem scope names (src/lib/rendering/PointRenderer.cu:770-886,1222,1252)
    for want in ("CountingPass", "CollectionPass", "SortingPass", "BlendingPass", "BlendBackwards"):
        assert any(want in n for n in names), want
    assert len(set(names)) == len(names) and "?" not in names


def test_null_arguments_are_refused_without_touching_a_gpu():
    lib = abi.load_library()
    assert lib.vetrast_create(None) == abi.ERR_INVALID_ARG
    assert lib.vetrast_forward(None, None, None) == abi.ERR_INVALID_ARG
    assert lib.vetrast_backward(None, None, None) == abi.ERR_INVALID_ARG
    assert lib.vetrast_set_profiling(None, 1) == abi.ERR_INVALID_ARG
    assert lib.vetrast_last_hip_error(None) == 0
    lib.vetrast_destroy(None)  # no-op


def test_product_path_has_no_cpu_fallback():
    """Without a GPU the host wrapper must raise instead of computing anything on the CPU."""
    import torch

    from vet_amd.rasterizer import Rasterizer

    if torch.cuda.is_available():
        pytest.skip("GPU present")
    with pytest.raises(RuntimeError):
        Rasterizer()


def test_product_sources_do_not_use_the_oracle():
    """The oracle is test infrastructure: nothing under vet_amd/ may import, load or link it."""
    pat = re.compile(r"from\s+oracle|import\s+oracle|oracle_py|libvetrast_oracle|vetref_|oracle/")
    for dirpath, _, files in os.walk(os.path.join(ROOT, "vet_amd")):
        for f in files:
            if f.endswith((".py", ".h", ".hip", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert not pat.search(text), os.path.join(dirpath, f)
