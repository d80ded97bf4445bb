"""Host-side checks of the C-ABI library that need no GPU: it loads, exports every symbol the
header declares, rejects bad arguments before touching the device, sizes the sort workspace
monotonically and builds the same camera matrices as the oracle."""
import ctypes
import os
import re

import numpy as np
import pytest

from flashgs_amd import cabi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "flashgs_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fgs_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(cabi.LIB_PATH)
    names = _declared_symbols()
    assert len(names) >= 12
    for name in names:
        assert hasattr(lib, name), "libflashgs_hip.so does not export %s" % name
        assert name in cabi.SIGNATURES, "flashgs_amd/cabi.py has no binding for %s" % name
    assert cabi.load().fgs_abi_version() == 2001       # FGS_ABI_VERSION of the header: major * 1000 + minor


def test_sort_buffer_size_is_monotonic_and_bounded():
    sizes = [cabi.get_sort_buffer_size(n) for n in (0, 1, 2047, 2048, 2049, 10 ** 6, 2 ** 27)]
    assert all(a <= b for a, b in zip(sizes, sizes[1:]))
    assert sizes[-1] >= 12 * 2 ** 27                     # room for the second key/value buffer
    assert sizes[-1] < 2.5 * 12 * 2 ** 27
    assert cabi.get_sort_buffer_size(-1) == 0
    assert cabi.get_sort_buffer_size(cabi.FGS_MAX_RENDERED) > 0


def test_camera_matrices_match_oracle_bit_for_bit(oracle):
    rng = np.random.default_rng(3)
    for k in range(20):
        q, _ = np.linalg.qr(rng.standard_normal((3, 3)))
        pos = rng.uniform(-30, 30, 3)
        W, H = int(rng.integers(64, 8000)), int(rng.integers(64, 4500))
        fx, fy = float(rng.uniform(100, 4000)), float(rng.uniform(100, 4000))
        a = cabi.camera_matrices(pos, q, W, H, fx, fy, 100.0, 0.01)
        b = oracle.view_proj(pos, q, W, H, fx, fy, 100.0, 0.01)
        assert np.array_equal(a[0].view(np.uint32), b[0].view(np.uint32))
        assert np.array_equal(a[1].view(np.uint32), b[1].view(np.uint32))


def _raises(code_fragment, fn, *args):
    with pytest.raises(RuntimeError) as e:
        fn(*args)
    assert code_fragment in str(e.value), str(e.value)


def test_bad_arguments_are_rejected_before_any_launch():
    cam = ([0, 0, 0], np.eye(3))
    # negative count, zero image, null buffers: all FGS_E_INVALID (-1)
    _raises("(-1)", cabi.preprocess, -1, 0, 0, 0, 0, 64, 64, 16, 16, cam[0], cam[1], 1.0, 1.0, 100.0, 0.01, 0, 0, 0, 0, 0, 0)
    _raises("(-1)", cabi.preprocess, 10, 0, 0, 0, 0, 0, 64, 16, 16, cam[0], cam[1], 1.0, 1.0, 100.0, 0.01, 0, 0, 0, 0, 0, 256)
    _raises("null", cabi.preprocess, 10, 0, 0, 0, 0, 64, 64, 16, 16, cam[0], cam[1], 1.0, 1.0, 100.0, 0.01, 0, 0, 0, 0, 0, 256)
    _raises("negative", cabi.sort_gaussian, -5, 64, 64, 16, 16, 256, 1 << 20, 256, 256, 256, 256)
    _raises("exceeds", cabi.sort_gaussian, 1 << 30, 64, 64, 16, 16, 256, 1 << 40, 256, 256, 256, 256)
    _raises("(-2)", cabi.sort_gaussian, 100000, 64, 64, 16, 16, 256, 1000, 256, 256, 256, 256)       # FGS_E_WORKSPACE
    _raises("aligned", cabi.sort_gaussian, 1000, 64, 64, 16, 16, 260, 1 << 30, 256, 256, 256, 256)
    _raises("unsupported", cabi.render_f32, 8, 8, 0, 64, 64, 0, 0, 0, 0, 0, 256, [0, 0, 0], 256, 0)
    _raises("null", cabi.render, 16, 16, 0, 64, 64, 0, 0, 0, 0, 0, 0, [0, 0, 0], 256)
    _raises("negative", cabi.render, 16, 16, -1, 64, 64, 0, 0, 0, 0, 0, 256, [0, 0, 0], 256)
    _raises("null", cabi.render, 16, 16, 5, 64, 64, 0, 0, 0, 0, 0, 256, [0, 0, 0], 256)
    with pytest.raises(ValueError):
        cabi.render(8, 8, 0, 64, 64, 0, 0, 0, 0, 0, 256, [0, 0, 0], 256)
    # an empty problem is fine and launches nothing
    cabi.sort_gaussian(0, 64, 64, 16, 16, 0, 0, 0, 0, 0, 0)
    cabi.preprocess(0, 0, 0, 0, 0, 64, 64, 16, 16, cam[0], cam[1], 1.0, 1.0, 100.0, 0.01, 0, 0, 0, 0, 0, 256)


def test_colour_sums_switch_round_trips_and_rejects_unknown_modes():
    prev = cabi.set_colour_sums(cabi.COLOUR_SUMS_FP32)
    try:
        assert prev == cabi.COLOUR_SUMS_FP32         # the library default is the reference's arithmetic
        assert cabi.set_colour_sums(cabi.COLOUR_SUMS_MATRIX_F16) == cabi.COLOUR_SUMS_FP32
        with pytest.raises(RuntimeError, match="unknown"):
            cabi.set_colour_sums(7)
        assert cabi.set_colour_sums(cabi.COLOUR_SUMS_MATRIX_F16) == cabi.COLOUR_SUMS_MATRIX_F16
    finally:
        cabi.set_colour_sums(prev)


def test_per_call_blend_flags_are_checked_on_the_host():
    # unknown bits and both modes at once are rejected before anything is launched
    for flags in (4, 8, cabi.BLEND_FP32 | cabi.BLEND_MATRIX_F16):
        _raises("(-1)", cabi.blend, 16, 16, 64, 64, 256, 256, 256, 256, 256, [0, 0, 0], 256, 0, 0, flags)
        _raises("(-1)", cabi.render_f32, 16, 16, 0, 64, 64, 0, 0, 0, 0, 0, 256, [0, 0, 0], 256, 0, 0, flags)
        assert cabi.blend_kernel_name(16, 16, 64, 64, flags) == ""


def test_wait_count_polls_a_host_word():
    """fgs_wait_count is host code: it returns what it finds in the word once that is not the
    pending mark (negative counts too), also when it arrives from elsewhere while it polls, and
    gives up with an error of its own after the time given."""
    import ctypes as C
    import threading
    word = C.c_int(12345)
    assert cabi.wait_count(C.addressof(word)) == 12345
    word.value = -2147483648
    assert cabi.wait_count(C.addressof(word)) == -2147483648
    word.value = cabi.COUNT_PENDING
    with pytest.raises(RuntimeError, match="no pair count within"):
        cabi.wait_count(C.addressof(word), 0.02)
    timer = threading.Timer(0.05, lambda: setattr(word, "value", 77))
    timer.start()
    assert cabi.wait_count(C.addressof(word), 5.0) == 77
    timer.join()
    with pytest.raises(RuntimeError, match="null"):
        cabi.wait_count(None)
