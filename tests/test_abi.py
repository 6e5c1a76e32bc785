"""CPU-only checks of the C-ABI boundary: the library loads, exports every symbol the header declares, the ctypes
mirrors have the C sizes, and host-side argument validation works without a GPU."""
import ctypes as C
import os
import re
import subprocess
import sys

import pytest

from trips_amd import _lib, abi, scenes

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "trips_splat.h")


def _declared_functions():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(trips_[a-z0-9_]+)\s*\(", src)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared_functions()
    assert len(names) >= 15
    for n in names:
        assert hasattr(lib, n), f"{n} declared in trips_splat.h but not exported"
    assert sorted(_lib.SYMBOLS) == names
    assert b"gfx950" in lib.trips_version()


def test_library_exports_every_unet_symbol():
    lib = _lib.load()
    src = open(os.path.join(ROOT, "include", "trips_unet.h")).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    names = sorted(set(re.findall(r"\b(trips_unet_[a-z0-9_]+)\s*\(", src)))
    assert names == sorted(_lib.UNET_SYMBOLS)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in trips_unet.h but not exported"


def test_unet_ctypes_mirrors_and_host_checks(tmp_path):
    prog = tmp_path / "sizes.c"
    prog.write_text('#include <stdio.h>\n#include "trips_unet.h"\nint main(){printf("%zu %zu %zu %zu\\n",'
                    "sizeof(TripsUnetDesc),sizeof(TripsUnetWeights),offsetof(TripsUnetDesc,level_w),"
                    "sizeof(TripsUnetGrads));return 0;}\n")
    exe = tmp_path / "sizes"
    subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), str(prog), "-o", str(exe)])
    got = [int(x) for x in subprocess.check_output([str(exe)]).split()]
    assert got == [C.sizeof(abi.TripsUnetDesc), C.sizeof(abi.TripsUnetWeights), abi.TripsUnetDesc.level_w.offset,
                   C.sizeof(abi.TripsUnetGrads)]
    lib = _lib.load()
    d = abi.make_unet_desc([16, 32, 64, 64], abi.layer_sizes(1920, 1080, 4))
    b, f = C.c_size_t(0), C.c_double(0)
    assert lib.trips_unet_workspace_size(C.byref(d), C.byref(b)) == 0
    assert b.value >= 960 * 540 * 32 * 2  # fp16 block outputs of the second level (the finest one's stay in its kernel)
    assert lib.trips_unet_flops(C.byref(d), C.byref(f)) == 0
    # two 3x3 convolutions per level, 2 flops per multiply-accumulate, plus the 1x1
    want = sum(2 * 2 * 9 * cin * cout * w * h for (cin, cout, (w, h)) in
               zip([32, 64, 64, 4], [12, 24, 56, 56], abi.layer_sizes(1920, 1080, 4))) + 2 * 16 * 3 * 1920 * 1080
    assert abs(f.value - want) < 1e-6 * want
    d.filters[0] = 200  # more convolution outputs than the kernels are built for
    assert lib.trips_unet_workspace_size(C.byref(d), C.byref(b)) == abi.TRIPS_ERR_UNSUPPORTED
    d = abi.make_unet_desc([16, 32], [(100, 60), (40, 30)])  # level 1 is not half of level 0
    assert lib.trips_unet_workspace_size(C.byref(d), C.byref(b)) == abi.TRIPS_ERR_UNSUPPORTED


def test_ctypes_mirrors_have_c_sizes(tmp_path):
    prog = tmp_path / "sizes.c"
    prog.write_text('#include <stdio.h>\n#include "trips_splat.h"\nint main(){printf("%zu %zu %zu %zu %zu %zu %zu\\n",'
                    "sizeof(TripsView),sizeof(TripsSplatDesc),sizeof(TripsSplatIn),sizeof(TripsSplatOut),"
                    "sizeof(TripsSplatGrads),sizeof(TripsAdamTensor),offsetof(TripsSplatDesc,views));return 0;}\n")
    exe = tmp_path / "sizes"
    subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), str(prog), "-o", str(exe)])
    got = [int(x) for x in subprocess.check_output([str(exe)]).split()]
    want = [C.sizeof(abi.TripsView), C.sizeof(abi.TripsSplatDesc), C.sizeof(abi.TripsSplatIn),
            C.sizeof(abi.TripsSplatOut), C.sizeof(abi.TripsSplatGrads), C.sizeof(abi.TripsAdamTensor),
            abi.TripsSplatDesc.views.offset]
    assert got == want


def test_header_compiles_as_c_and_cpp(tmp_path):
    for comp, ext in (("gcc", "c"), ("g++", "cpp")):
        src = tmp_path / f"t.{ext}"
        src.write_text('#include "trips_splat.h"\nint main(void){return TRIPS_ABI_VERSION - 2;}\n')
        subprocess.check_call([comp, "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), "-c", str(src), "-o",
                               str(tmp_path / "t.o")])


def _rc(fn, *a):
    return fn(*a)


def test_size_queries_and_layer_sizes_host_only():
    lib = _lib.load()
    sc = scenes.tiny(n=100, w=1245, h=825, num_layers=8)
    for fl in (False, True):
        d = abi.desc_for_scene(sc, floor_layer_sizes=fl)
        w = (C.c_int32 * 8)()
        h = (C.c_int32 * 8)()
        assert lib.trips_splat_layer_sizes(C.byref(d), w, h) == 0
        assert list(zip(w, h)) == abi.layer_sizes(1245, 825, 8, fl)
    d = abi.desc_for_scene(sc)
    ws, sv = C.c_size_t(0), C.c_size_t(0)
    assert lib.trips_splat_workspace_size(C.byref(d), C.byref(ws)) == 0
    assert lib.trips_splat_saved_size(C.byref(d), C.byref(sv)) == 0
    _, _, P = abi.pyramid_pixels(d)
    assert ws.value >= 100 * 8 * (8 + 8) + 2 * P * 4  # worst case: a key and a bin entry per (point, layer) + counters
    assert sv.value >= P * d.list_depth * 4 + 100 * 64
    # a capped list storage shrinks the forward's share of the workspace (eval mode has no backward share)
    ws1, ws2 = C.c_size_t(0), C.c_size_t(0)
    sc_big = scenes.tiny(n=100_000, w=64, h=48, num_layers=8)
    assert lib.trips_splat_workspace_size(C.byref(abi.desc_for_scene(sc_big, train=False)), C.byref(ws1)) == 0
    assert lib.trips_splat_workspace_size(C.byref(abi.desc_for_scene(sc_big, train=False, max_list_entries=1000)),
                                          C.byref(ws2)) == 0
    assert ws2.value < ws1.value and ws1.value >= 100_000 * 8 * (8 + 8)
    # two views double the saved state
    sc2 = scenes.tiny(n=100, w=64, h=48, num_layers=3, views=2)
    sc1 = scenes.tiny(n=100, w=64, h=48, num_layers=3, views=1)
    a, b = C.c_size_t(0), C.c_size_t(0)
    lib.trips_splat_saved_size(C.byref(abi.desc_for_scene(sc1)), C.byref(a))
    lib.trips_splat_saved_size(C.byref(abi.desc_for_scene(sc2)), C.byref(b))
    assert b.value == 2 * a.value


@pytest.mark.parametrize("field,value,code", [
    ("abi_version", 99, abi.TRIPS_ERR_INVALID_ARG),
    ("num_layers", 0, abi.TRIPS_ERR_INVALID_ARG),
    ("num_layers", 9, abi.TRIPS_ERR_INVALID_ARG),
    ("list_depth", 12, abi.TRIPS_ERR_UNSUPPORTED),
    ("num_channels", 5, abi.TRIPS_ERR_UNSUPPORTED),
    ("num_views", 0, abi.TRIPS_ERR_INVALID_ARG),
    ("num_views", 17, abi.TRIPS_ERR_INVALID_ARG),
    ("num_points", -1, abi.TRIPS_ERR_INVALID_ARG),
    ("layout", 7, abi.TRIPS_ERR_INVALID_ARG),
    ("background_mode", 2, abi.TRIPS_ERR_INVALID_ARG),
    ("max_list_entries", -5, abi.TRIPS_ERR_INVALID_ARG),
])
def test_descriptor_validation(field, value, code):
    lib = _lib.load()
    sc = scenes.tiny(n=100)
    d = abi.desc_for_scene(sc)
    setattr(d, field, value)
    b = C.c_size_t(0)
    assert lib.trips_splat_workspace_size(C.byref(d), C.byref(b)) == code
    msg = lib.trips_last_error_string().decode()
    assert msg, "an error must leave a message"


def test_view_validation_and_null_arguments():
    lib = _lib.load()
    sc = scenes.tiny(n=100, views=2)
    b = C.c_size_t(0)
    d = abi.desc_for_scene(sc)
    d.views[1].w += 1
    assert lib.trips_splat_workspace_size(C.byref(d), C.byref(b)) == abi.TRIPS_ERR_INVALID_ARG
    d = abi.desc_for_scene(sc)
    d.views[0].camera_model_type = 1  # OCAM: not on this path
    assert lib.trips_splat_workspace_size(C.byref(d), C.byref(b)) == abi.TRIPS_ERR_UNSUPPORTED
    d = abi.desc_for_scene(sc)
    d.views[1].image_index = 5
    assert lib.trips_splat_workspace_size(C.byref(d), C.byref(b)) == abi.TRIPS_ERR_INVALID_ARG
    d = abi.desc_for_scene(sc)
    assert lib.trips_splat_workspace_size(None, C.byref(b)) == abi.TRIPS_ERR_INVALID_ARG
    assert lib.trips_splat_workspace_size(C.byref(d), None) == abi.TRIPS_ERR_INVALID_ARG
    # entry points reject a NULL context before touching the device
    tin, out, grads = abi.TripsSplatIn(), abi.TripsSplatOut(), abi.TripsSplatGrads()
    assert lib.trips_splat_forward(None, C.byref(d), C.byref(tin), C.byref(out), None, 0, None) == abi.TRIPS_ERR_INVALID_ARG
    arr = (C.c_void_p * 8)()
    assert lib.trips_splat_backward(None, C.byref(d), C.byref(tin), None, arr, C.byref(grads), None, 0,
                                    None) == abi.TRIPS_ERR_INVALID_ARG
    assert lib.trips_adam_step_fused(None, None, 0, None) == abi.TRIPS_ERR_INVALID_ARG
    assert lib.trips_apply_tangent(None, None, None, 0, None) == abi.TRIPS_ERR_INVALID_ARG
    assert lib.trips_profile_enable(None, 1) == abi.TRIPS_ERR_INVALID_ARG


def test_packed_adam_state_size_host_only():
    """Rows of the packed optimiser state: 12 bytes per element of a point (6 + C of them), whole 128-byte lines."""
    lib = _lib.load()
    for c, row in ((3, 128), (4, 128), (6, 256), (8, 256), (16, 384)):
        b, r = C.c_size_t(0), C.c_int(0)
        assert lib.trips_adam_points_state_size(1000, c, C.byref(b), C.byref(r)) == 0
        assert r.value == row and b.value == 1000 * row and 12 * (6 + c) <= row
    b = C.c_size_t(0)
    assert lib.trips_adam_points_state_size(10, 5, C.byref(b), None) == abi.TRIPS_ERR_UNSUPPORTED
    assert lib.trips_adam_points_state_size(-1, 4, C.byref(b), None) == abi.TRIPS_ERR_INVALID_ARG
    assert lib.trips_adam_points_state_size(10, 4, None, None) == abi.TRIPS_ERR_INVALID_ARG
    assert lib.trips_adam_step_points(None, None, 10, 4, None, None) == abi.TRIPS_ERR_INVALID_ARG


def test_too_many_points_for_32_bit_offsets():
    lib = _lib.load()
    sc = scenes.tiny(n=10)
    d = abi.desc_for_scene(sc)
    d.num_points = 300_000_000  # N*L = 2.4e9 (point, layer) pairs exceed 2^31-1 with 8 layers
    d.num_layers = 8
    b = C.c_size_t(0)
    assert lib.trips_splat_workspace_size(C.byref(d), C.byref(b)) == abi.TRIPS_ERR_UNSUPPORTED
    # a granted capacity does not shorten the 32-bit prefix sums over the pairs that could exist: still refused
    d.max_list_entries = 1_000_000_000
    assert lib.trips_splat_workspace_size(C.byref(d), C.byref(b)) == abi.TRIPS_ERR_UNSUPPORTED
    d.num_points = 250_000_000  # N*L = 2.0e9 fits: one key and one bin entry per pair, the four list entries of a
    assert lib.trips_splat_workspace_size(C.byref(d), C.byref(b)) == 0  # pair are only counted (in 64 bits)


def test_abi_version_mismatch_is_refused():
    lib = _lib.load()
    sc = scenes.tiny(n=10)
    d = abi.desc_for_scene(sc)
    b = C.c_size_t(0)
    assert lib.trips_splat_workspace_size(C.byref(d), C.byref(b)) == 0
    d.abi_version = abi.TRIPS_ABI_VERSION - 1  # a caller built against the previous header
    assert lib.trips_splat_workspace_size(C.byref(d), C.byref(b)) == abi.TRIPS_ERR_INVALID_ARG
    assert lib.trips_splat_saved_size(C.byref(d), C.byref(b)) == abi.TRIPS_ERR_INVALID_ARG
    assert b"abi_version" in lib.trips_last_error_string()


def test_check_needs_a_workspace():
    lib = _lib.load()
    # (no context is dereferenced before the arguments are looked at)
    assert lib.trips_splat_check(None, None, None) == abi.TRIPS_ERR_INVALID_ARG
    assert lib.trips_splat_check_static(None, None) == abi.TRIPS_ERR_INVALID_ARG


def test_product_path_fails_loudly_without_gpu_or_library(monkeypatch, tmp_path):
    import torch
    from trips_amd import renderer
    if not torch.cuda.is_available():
        with pytest.raises(RuntimeError):
            renderer.SplatContext(0)
    # a missing library is an error, not a silent fallback
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _lib.load()


def test_product_code_does_not_touch_the_oracle():
    # nothing under trips_amd/, include/ or bench-independent product code may reference oracle/
    bad = []
    for base in ("trips_amd", "include"):
        for dirpath, _, files in os.walk(os.path.join(ROOT, base)):
            for f in files:
                if f.endswith((".py", ".h", ".hip", ".cpp")):
                    text = open(os.path.join(dirpath, f), errors="ignore").read()
                    if "oracle" in text.lower():
                        bad.append(os.path.join(dirpath, f))
    assert not bad, bad
