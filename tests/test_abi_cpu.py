"""The C-ABI library loads without a GPU, exports what include/moodist_hip.h declares, and
rejects bad arguments before any launch.  No compute calls here."""

import ctypes
import os
import re

import pytest

from moodist_amd import _abi as abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "moodist_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mdh_[a-z_0-9]+)\s*\(", text)))


def test_every_declared_symbol_is_exported():
    L = abi.lib()
    names = declared_symbols()
    assert set(names) == set(abi.SYMBOLS)
    for n in names:
        assert getattr(L, n) is not None


def test_abi_version_and_error_strings():
    L = abi.lib()
    assert L.mdh_abi_version() == abi.ABI_VERSION
    assert L.mdh_error_string(0) == b"success"
    assert L.mdh_error_string(2) == b"Unsupported dtype for reduce operation"
    assert L.mdh_error_string(3) == b"Unsupported reduce operation"


def test_box_struct_layout_matches_header():
    # const void*, void*, int32, int32, 3 x int64[10]
    assert ctypes.sizeof(abi.Box) == 8 + 8 + 4 + 4 + 3 * 8 * abi.MAX_DIMS


@pytest.mark.parametrize("call,match", [
    (lambda: abi.reduce([], 0, 16, 4, abi.DTYPE_FLOAT32, abi.OP_SUM), "nsrc 0 outside"),
    (lambda: abi.reduce([16] * 65, 0, 16, 4, abi.DTYPE_FLOAT32, abi.OP_SUM), "nsrc 65 outside"),
    (lambda: abi.reduce([16, 32], 2, 48, 4, abi.DTYPE_FLOAT32, abi.OP_SUM), "first 2 outside"),
    (lambda: abi.reduce([16], 0, 32, 4, 0, abi.OP_SUM), "Unsupported dtype for reduce operation"),
    (lambda: abi.reduce([16], 0, 32, 4, abi.DTYPE_FLOAT32, 2), "Unsupported reduce operation"),
    (lambda: abi.reduce([16], 0, 32, 4, abi.DTYPE_INT32, abi.OP_AVG), "Unsupported reduce operation"),
    (lambda: abi.reduce([16], 0, 32, 4, abi.DTYPE_INT64, abi.OP_PREMUL_SUM), "Unsupported reduce operation"),
    (lambda: abi.reduce([0], 0, 32, 4, abi.DTYPE_FLOAT32, abi.OP_SUM), "source 0 is null"),
    (lambda: abi.reduce([16], 0, 0, 4, abi.DTYPE_FLOAT32, abi.OP_SUM), "null pointer"),
    (lambda: abi.reduce([18], 0, 64, 4, abi.DTYPE_FLOAT32, abi.OP_SUM), "not aligned to its element size"),
    (lambda: abi.reduce([64], 0, 72, 4, abi.DTYPE_FLOAT32, abi.OP_SUM), "partially overlaps"),
    (lambda: abi.gather([16], 1024, 8, 2, 4, 8, 64), "row pitch is smaller"),
    (lambda: abi.gather([16, 32], 1024, 8, 2, 8, 8, 8), "shards would overlap"),
    (lambda: abi.gather([0], 1024, 8, 1, 8, 8, 8), "source 0 is null"),
    (lambda: abi.gather([16], 1024, 8, 2 ** 30, 2 ** 40, 8, 8), "not a plausible device size"),
    (lambda: abi.gather([16, 32], 1024, 8, 1, 8, 8, 2 ** 60), "not a plausible device size"),
    (lambda: abi.copy_boxes([abi.make_box(16, 32, [4], [1], [1])], 3), "itemsize 3"),
    (lambda: abi.copy_boxes([abi.make_box(0, 32, [4], [1], [1])], 4), "null pointer"),
    (lambda: abi.copy_boxes([abi.make_box(16, 32, [4], [-1], [1])], 4), "negative extent or stride"),
    (lambda: abi.copy_boxes([abi.make_box(18, 32, [4], [1], [1])], 4), "not aligned to its element size"),
    (lambda: abi.copy_boxes([abi.make_box(16, 32, [4, 4], [2 ** 50, 1], [4, 1])], 4), "spans more than a plausible device size"),
    # five strided extents that cannot merge, the slowest ones huge: the host would have to cut
    # the box into 2^24 pieces
    (lambda: abi.copy_boxes([abi.make_box(16, 1 << 40, [4096, 4096, 2, 2, 2, 1], [2 ** 22, 2 ** 10, 64, 16, 4, 1],
                                          [2 ** 24, 2 ** 11, 128, 32, 8, 1])], 1), "more than 1048576 pieces"),
    (lambda: abi.reduce_many([([16], 0, 32, 4), ([16, 48], 2, 64, 4)], abi.DTYPE_FLOAT32, abi.OP_SUM), r"first 2 outside 0..1 \(job 1\)"),
    (lambda: abi.reduce_many([([16], 0, 32, 4), ([0], 0, 64, 4)], abi.DTYPE_FLOAT32, abi.OP_SUM), r"source 0 is null \(job 1\)"),
    (lambda: abi.reduce_many([([16], 0, 32, 4)], 11, abi.OP_SUM), "Unsupported dtype"),
    (lambda: abi.reduce_many([([16], 0, 32, 4)], abi.DTYPE_INT32, abi.OP_AVG), "Unsupported reduce operation"),
    (lambda: abi.reduce_many([([16] * 65, 0, 32, 4)], abi.DTYPE_FLOAT32, abi.OP_SUM), "nsrc 65 outside"),
    (lambda: abi.reduce_many([([64], 0, 68, 4)], abi.DTYPE_FLOAT32, abi.OP_SUM), "partially overlaps"),
    (lambda: abi.allreduce_many([([16, 48], 2, 0, 4)], abi.DTYPE_FLOAT32, abi.OP_SUM), r"first 2 outside 0..1 \(job 0\)"),
    (lambda: abi.allreduce_many([([64, 72], 0, 0, 4)], abi.DTYPE_FLOAT32, abi.OP_SUM), r"overlaps source 1 \(job 0\)"),
    (lambda: abi.allreduce_many([([64, 128, 64], 0, 0, 4)], abi.DTYPE_FLOAT32, abi.OP_SUM), r"sources 0 and 2 overlap"),
    (lambda: abi.allreduce_many([([64, 128], 0, 0, 4)], abi.DTYPE_INT64, abi.OP_PREMUL_SUM), "Unsupported reduce operation"),
    (lambda: abi.set_tuning("reduce_wg_per_cu", 10), "does not take 10"),
    (lambda: abi.set_tuning("no_such_knob", 1), "unknown knob"),
    (lambda: abi.set_tuning("reduce_unroll", 3), "does not take 3"),
    (lambda: abi.set_tuning("box_preload", 2), "does not take 2"),
])
def test_bad_arguments_are_refused_before_launch(call, match):
    with pytest.raises(abi.MoodistError, match=match):
        call()


def test_empty_work_is_a_no_op_without_a_device():
    abi.reduce([16], 0, 32, 0, abi.DTYPE_FLOAT32, abi.OP_SUM)  # numel == 0
    abi.reduce_many([], abi.DTYPE_FLOAT32, abi.OP_SUM)
    abi.reduce_many([([16], 0, 32, 0), ([16, 48], 1, 64, 0)], abi.DTYPE_BFLOAT16, abi.OP_MAX)
    abi.gather([16], 1024, 0, 1, 0, 0, 0)
    abi.gather([], 1024, 8, 1, 8, 8, 8)
    abi.copy_boxes([], 4)
    abi.copy_boxes([abi.make_box(16, 32, [4, 0], [1, 1], [1, 1])], 4)


def test_tuning_round_trip():
    old = abi.get_tuning("copy_unroll")
    abi.set_tuning("copy_unroll", 2)
    assert abi.get_tuning("copy_unroll") == 2
    abi.set_tuning("copy_unroll", old)
    assert abi.get_tuning("box_preload") == 0
    abi.set_tuning("box_preload", 1)
    assert abi.get_tuning("box_preload") == 1
    abi.set_tuning("box_preload", 0)


def test_missing_kernel_library_fails_loudly(monkeypatch, tmp_path):
    # there is no CPU fallback: without the built library every entry raises
    monkeypatch.setattr(abi, "_lib", None)
    monkeypatch.setattr(abi, "LIB_PATH", str(tmp_path / "libmoodist_hip.so"))
    with pytest.raises(abi.MoodistError, match="is not built"):
        abi.reduce([16], 0, 32, 4, abi.DTYPE_FLOAT32, abi.OP_SUM)
    with pytest.raises(abi.MoodistError, match="is not built"):
        abi.gather([16], 32, 4, 1, 4, 4, 4)


def test_product_code_never_imports_the_oracle():
    import glob

    for path in glob.glob(os.path.join(ROOT, "moodist_amd", "**", "*"), recursive=True):
        if os.path.isfile(path) and path.endswith((".py", ".cc", ".h", ".hip", ".sh")):
            text = open(path, errors="ignore").read()
            assert "import oracle" not in text and "from oracle" not in text and "liboracle" not in text, path


def test_launch_without_a_device_is_an_error_not_a_crash():
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present; this checks the no-device error path")
    with pytest.raises(abi.MoodistError, match="launch failed"):
        abi.reduce([4096, 8192], 0, 16384, 64, abi.DTYPE_FLOAT32, abi.OP_SUM)
    with pytest.raises(abi.MoodistError, match="launch failed"):
        abi.gather([4096], 16384, 64, 1, 64, 64, 64)
    with pytest.raises(abi.MoodistError, match="launch failed"):
        abi.reduce_many([([4096, 8192], 0, 16384, 64), ([4096], 0, 32768, 3)], abi.DTYPE_FLOAT32, abi.OP_SUM)
