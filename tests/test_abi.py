"""The C-ABI library loads and exports every entry point the public header declares (no GPU needed)."""

from __future__ import annotations

import ctypes
import os
import re

import pytest

from conftest import ROOT


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "gradoom_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gd_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = _declared_functions()
    for required in ("gd_renderer_create", "gd_renderer_destroy", "gd_render", "gd_observe", "gd_expand_rgb24", "gd_version"):
        assert required in names


def test_library_exports_every_declared_symbol():
    from gradoom_amd import _build, _lib

    if not os.path.exists(_build.LIBRARY):
        pytest.skip("libgradoom_amd.so not built (run __graft_entry__.build())")
    lib = ctypes.CDLL(_build.LIBRARY)
    missing = [name for name in _declared_functions() if not hasattr(lib, name)]
    assert not missing, missing
    assert set(_declared_functions()) == set(_lib.SYMBOLS)
    lib.gd_version.restype = ctypes.c_char_p
    assert b"gfx950" in lib.gd_version()


def test_struct_layouts_match_header_field_order():
    from gradoom_amd import _abi

    text = open(os.path.join(ROOT, "include", "gradoom_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)

    def fields(struct_name):
        body = re.search(r"typedef struct " + struct_name + r" \{(.*?)\} " + struct_name + ";", text, flags=re.S).group(1)
        names = []
        for statement in body.split(";"):
            statement = statement.strip()
            if not statement:
                continue
            declarators = statement.split(",")
            first = declarators[0].split()[-1]
            names.append(first.lstrip("*"))
            names += [d.strip().lstrip("*") for d in declarators[1:]]
        return names

    assert fields("gd_map_desc") == [name for name, _ in _abi.MapDesc._fields_]
    assert fields("gd_lanes_desc") == [name for name, _ in _abi.LanesDesc._fields_]
    assert fields("gd_frame_out") == [name for name, _ in _abi.FrameOut._fields_]
    assert fields("gd_overlay_desc") == [name for name, _ in _abi.OverlayDesc._fields_]
    assert fields("gd_actor_desc") == [name for name, _ in _abi.ActorDesc._fields_]
    assert fields("gd_weapon_desc") == [name for name, _ in _abi.WeaponDesc._fields_]


def test_struct_sizes_match_what_a_c_compiler_makes_of_the_header(tmp_path):
    # the size every descriptor announces in struct_size is the size gcc gives the header's struct
    import subprocess

    from gradoom_amd import _abi

    source = tmp_path / "sizes.c"
    source.write_text(
        '#include <stdio.h>\n#include "gradoom_amd.h"\nint main(void) { printf("%zu %zu %zu %zu %zu %zu %d\\n", sizeof(gd_map_desc), '
        "sizeof(gd_lanes_desc), sizeof(gd_frame_out), sizeof(gd_overlay_desc), sizeof(gd_actor_desc), sizeof(gd_weapon_desc), GD_ABI_VERSION); return 0; }\n"
    )
    binary = tmp_path / "sizes"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(source), "-o", str(binary)], check=True)
    sizes = [int(v) for v in subprocess.run([str(binary)], check=True, capture_output=True, text=True).stdout.split()]
    ours = [ctypes.sizeof(t) for t in (_abi.MapDesc, _abi.LanesDesc, _abi.FrameOut, _abi.OverlayDesc, _abi.ActorDesc, _abi.WeaponDesc)]
    assert sizes[:6] == ours
    assert sizes[6] == _abi.ABI_VERSION
    assert _abi.LanesDesc().struct_size == ours[1]


def _create(tables):
    """gd_renderer_create on host tables; returns the exception class the binding maps the code to (or None).

    Every check exercised here runs on the host before the first HIP call, so this needs no GPU."""

    import numpy as np

    from gradoom_amd import _abi, _build, _lib

    if not os.path.exists(_build.LIBRARY):
        pytest.skip("libgradoom_amd.so not built (run __graft_entry__.build())")
    lib = _lib.library()
    desc, keep = _abi.host_map_desc(tables)
    cosine = np.ones(320, dtype=np.float32)
    handle = ctypes.c_void_p()
    return lib, desc, keep, cosine, handle


@pytest.fixture(scope="module")
def small_tables():
    from gradoom_amd import mapbuild, synthmap

    return mapbuild.build_map_tables(synthmap.generate_map(31, grid=(4, 3), sectors=10, linedefs=48))


def test_create_refuses_a_descriptor_of_another_header_version(small_tables):
    from gradoom_amd import _lib

    lib, desc, keep, cosine, handle = _create(small_tables)
    desc.struct_size -= 8
    with pytest.raises(ValueError, match="struct_size"):
        _lib.check(lib.gd_renderer_create(ctypes.byref(desc), cosine.ctypes.data, 4, ctypes.byref(handle)))
    assert not handle.value


@pytest.mark.parametrize(
    "field, index, value, message",
    [
        ("wall_sectors", (5, 0), 99, "wall_sectors"),
        ("wall_sectors", (5, 1), -2, "wall_sectors"),
        ("side_tex", (2, 0, 1), 4096, "side_tex"),
        ("sector_floor_tex", (1,), -1, "flat"),
        ("wall_vertex", (7, 1), 100000, "wall_vertex"),
        ("vertex_wall_idx", (0,), 48, "vertex_wall"),
        ("sector_edge_ofs", (2,), 0, "sector_edge_ofs"),
        ("tex_w", (0,), 0, "texture size"),
    ],
)
def test_create_refuses_indices_outside_their_tables(small_tables, field, index, value, message):
    from gradoom_amd import _lib

    tables = dict(small_tables)
    array = tables[field].copy()
    array[index] = value
    tables[field] = array
    lib, desc, keep, cosine, handle = _create(tables)
    with pytest.raises(ValueError, match=message):
        _lib.check(lib.gd_renderer_create(ctypes.byref(desc), cosine.ctypes.data, 4, ctypes.byref(handle)))
