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
