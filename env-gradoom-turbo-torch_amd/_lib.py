"""ctypes binding of ``libgradoom_amd.so`` (the C ABI of ``include/gradoom_amd.h``).

There is no fallback: if the shared library is missing or does not export every
symbol of the header, importing this module raises.
"""

from __future__ import annotations

import ctypes as C
import os

from . import _abi, _build

SYMBOLS = (
    "gd_version",
    "gd_abi_version",
    "gd_last_error",
    "gd_renderer_create",
    "gd_renderer_destroy",
    "gd_renderer_status",
    "gd_renderer_scribble",
    "gd_renderer_set_assembly",
    "gd_renderer_set_sector_lights",
    "gd_renderer_set_overlays",
    "gd_render",
    "gd_render_static",
    "gd_render_timed",
    "gd_observe",
    "gd_expand_rgb24",
    "gd_pack_actors",
    "gd_pack_weapon",
)

_LIBRARY = None


def library() -> C.CDLL:
    global _LIBRARY
    if _LIBRARY is not None:
        return _LIBRARY
    path = _build.LIBRARY
    if not os.path.exists(path):
        raise RuntimeError(
            f"{path} is missing: run `python -c 'import __graft_entry__ as e; e.build()'` to compile the HIP kernels"
        )
    lib = C.CDLL(path)
    missing = [name for name in SYMBOLS if not hasattr(lib, name)]
    if missing:
        raise RuntimeError(f"{path} does not export {missing}")
    lib.gd_version.restype = C.c_char_p
    lib.gd_abi_version.restype = C.c_uint32
    if lib.gd_abi_version() != _abi.ABI_VERSION:
        raise RuntimeError(
            f"{path} was built with struct layout version {lib.gd_abi_version()}, this package expects {_abi.ABI_VERSION}: rebuild it"
        )
    lib.gd_last_error.restype = C.c_char_p
    lib.gd_renderer_create.restype = C.c_int
    lib.gd_renderer_create.argtypes = [C.POINTER(_abi.MapDesc), C.c_void_p, C.c_int32, C.POINTER(C.c_void_p)]
    lib.gd_renderer_destroy.restype = None
    lib.gd_renderer_destroy.argtypes = [C.c_void_p]
    lib.gd_renderer_status.restype = C.c_int
    lib.gd_renderer_status.argtypes = [C.c_void_p, C.POINTER(C.c_int32)]
    lib.gd_renderer_set_assembly.restype = C.c_int
    lib.gd_renderer_set_assembly.argtypes = [C.c_void_p, C.c_int32]
    lib.gd_renderer_scribble.restype = C.c_int
    lib.gd_renderer_scribble.argtypes = [C.c_void_p, C.c_int32, C.c_void_p]
    lib.gd_renderer_set_overlays.restype = C.c_int
    lib.gd_renderer_set_overlays.argtypes = [C.c_void_p, C.POINTER(_abi.OverlayDesc)]
    lib.gd_renderer_set_sector_lights.restype = C.c_int
    lib.gd_renderer_set_sector_lights.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
    lib.gd_render.restype = C.c_int
    lib.gd_render.argtypes = [C.c_void_p, C.POINTER(_abi.LanesDesc), C.POINTER(_abi.FrameOut), C.c_void_p]
    lib.gd_render_static.restype = C.c_int
    lib.gd_render_static.argtypes = [C.c_void_p, C.POINTER(_abi.LanesDesc), C.POINTER(_abi.FrameOut), C.c_void_p]
    lib.gd_render_timed.restype = C.c_int
    lib.gd_render_timed.argtypes = [
        C.c_void_p, C.POINTER(_abi.LanesDesc), C.POINTER(_abi.FrameOut), C.c_void_p, C.c_int32, C.POINTER(C.c_float), C.c_int32,
    ]
    lib.gd_observe.restype = C.c_int
    lib.gd_observe.argtypes = [C.c_void_p, C.c_int32, C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p]
    lib.gd_expand_rgb24.restype = C.c_int
    lib.gd_expand_rgb24.argtypes = [C.c_void_p, C.c_int32, C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p]
    lib.gd_pack_actors.restype = C.c_int
    lib.gd_pack_actors.argtypes = [C.POINTER(_abi.ActorDesc), C.c_void_p]
    lib.gd_pack_weapon.restype = C.c_int
    lib.gd_pack_weapon.argtypes = [C.POINTER(_abi.WeaponDesc), C.c_void_p]
    _LIBRARY = lib
    return lib


def check(code: int) -> None:
    """Translate a negative return code into the exception class the reference would raise."""

    if code == _abi.GD_OK:
        return
    message = library().gd_last_error().decode(errors="replace")
    if code == _abi.GD_E_ARG:
        raise ValueError(message)
    if code == _abi.GD_E_UNSUPPORTED:
        raise NotImplementedError(message)
    raise RuntimeError(f"gradoom_amd error {code}: {message}")
