"""The plugin entry of libmoodist.so (include/moodist_plugin.h), checked on the built library
without a GPU: the one symbol the reference's wrapper resolves (wrapper/moodist_loader.cc:363-386),
its version/magic handshake, the table's layout against the reference's own header, and
rank / size / options called through the table's slots.  No compute calls.
"""

import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "moodist_amd", "libmoodist.so")
HEADER = os.path.join(ROOT, "include", "moodist_plugin.h")
REFERENCE_HEADER = "/root/reference/api/moodist_api.h"
API_VERSION = 2
SOURCE_TREE_MAGIC = 0x4D49333535584D44  # what a translation unit compiled on its own carries


def build_magic():
    """The number the built libmoodist.so drew (moodist_amd/csrc/build_host.sh)."""
    L = ctypes.CDLL(LIB)
    L.moodist_build_magic.restype = ctypes.c_uint64
    return L.moodist_build_magic()


def struct_members(text, name):
    """Member names of `struct name { ... };` in declaration order: function pointers
    `(*member)(...)` and comma lists of OffPath members."""
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    body = text[text.index("struct %s {" % name):]
    body = body[body.index("{") + 1:body.index("\n};")]
    names = []
    for statement in body.split(";"):
        statement = statement.strip()
        if not statement:
            continue
        if statement.startswith("OffPath"):
            names += [n.strip() for n in statement[len("OffPath"):].split(",")]
            continue
        m = re.search(r"\(\*\s*(\w+)\s*\)\s*\(", statement)
        if m:
            names.append(m.group(1))
        elif re.match(r"uint64_t\s+magic$", statement):
            names.append("magic")
    return names


def own_members(name):
    return struct_members(open(HEADER).read(), name)


def slot_offset(member):
    names = own_members("CoreApi")
    assert names[0] == "magic"
    return 8 + 8 * (names.index(member) - 1)


@pytest.fixture(scope="module")
def lib():
    L = ctypes.CDLL(LIB)
    L.moodistGetApi.restype = ctypes.c_void_p
    L.moodistGetApi.argtypes = [ctypes.c_uint32, ctypes.c_void_p]
    return L


@pytest.fixture(scope="module")
def wrapper_table():
    # 38 slots; the only callback this test's calls reach is cudaCurrentDevice (slot 0)
    names = own_members("WrapperApi")
    assert len(names) == 38 and names[0] == "cudaCurrentDevice"
    current_device = ctypes.CFUNCTYPE(ctypes.c_int)(lambda: 0)
    table = (ctypes.c_void_p * 38)()
    table[0] = ctypes.cast(current_device, ctypes.c_void_p).value
    return table, current_device  # the callback object must outlive the table


def test_only_the_documented_entry_points_are_exported():
    import subprocess

    out = subprocess.run(["nm", "-D", "--defined-only", LIB], check=True, capture_output=True, text=True).stdout
    mine = sorted(l.split()[-1] for l in out.splitlines() if " T " in l)
    assert "moodistGetApi" in mine
    assert all(n.startswith("moodist") for n in mine), mine


def test_version_mismatch_gives_null_and_the_table_carries_the_build_magic(lib, wrapper_table):
    table, _ = wrapper_table
    for wrong in (0, 1, API_VERSION + 1, 0xFFFFFFFF):
        assert lib.moodistGetApi(wrong, table) is None
    api = lib.moodistGetApi(API_VERSION, table)
    assert api
    assert ctypes.c_uint64.from_address(api).value == build_magic()
    assert build_magic() != SOURCE_TREE_MAGIC and build_magic() != 0  # drawn by the build, not the header's constant
    # one table per core: asking again gives the same one
    assert lib.moodistGetApi(API_VERSION, table) == api


def test_table_has_the_reference_slot_order():
    mine = own_members("CoreApi")
    assert len(mine) == 1 + 69
    assert len(own_members("WrapperApi")) == 38
    # the hot path's slots, by the reference's names
    for n in ("createProcessGroup", "processGroupDestroy", "processGroupRank", "processGroupSize",
              "processGroupGetOption", "processGroupSetOption", "processGroupAllGather",
              "processGroupReduceScatter", "processGroupAllreduce", "compileOpFull", "customOpCall",
              "customOpDestroy", "futureWait", "futureDestroy"):
        assert n in mine
    if not os.path.exists(REFERENCE_HEADER):
        pytest.skip("the reference's header is not on this machine")
    text = open(REFERENCE_HEADER).read()
    # the reference declares `void (*deleter)(void* ctx)` as a parameter inside one member
    theirs = [n for n in struct_members(text, "CoreApi")]
    assert mine == theirs
    theirs_w = [n for n in struct_members(text, "WrapperApi") if n != "deleter"]
    assert own_members("WrapperApi") == theirs_w


def test_rank_size_and_options_through_the_table(lib, wrapper_table):
    table, _ = wrapper_table
    api = lib.moodistGetApi(API_VERSION, table)

    def slot(member, restype, *argtypes):
        address = ctypes.c_void_p.from_address(api + slot_offset(member)).value
        return ctypes.CFUNCTYPE(restype, *argtypes)(address)

    # api::ProcessGroupHandle createProcessGroup(void* store, int rank, int size): the handle is one
    # pointer wide and not trivially destructible, so it comes back through a hidden first argument
    create = slot("createProcessGroup", ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p,
                  ctypes.c_int, ctypes.c_int)
    destroy = slot("processGroupDestroy", None, ctypes.c_void_p)
    rank = slot("processGroupRank", ctypes.c_int, ctypes.c_void_p)
    size = slot("processGroupSize", ctypes.c_int, ctypes.c_void_p)
    get_option = slot("processGroupGetOption", ctypes.c_int64, ctypes.c_void_p, ctypes.c_char_p)
    set_option = slot("processGroupSetOption", None, ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int64)
    get_pkl = slot("processGroupGetPreferKernelLess", ctypes.c_bool, ctypes.c_void_p)
    set_pkl = slot("processGroupSetPreferKernelLess", None, ctypes.c_void_p, ctypes.c_bool)

    store = ctypes.create_string_buffer(8)  # its address names the world
    groups = []
    for r in range(3):
        out = ctypes.c_void_p()
        create(ctypes.byref(out), ctypes.addressof(store), r, 3)
        assert out.value
        # ApiRefCounted: the object starts with its reference count, 1 for the handle just returned
        assert ctypes.c_size_t.from_address(out.value).value == 1
        groups.append(out.value)
    assert [rank(g) for g in groups] == [0, 1, 2]
    assert [size(g) for g in groups] == [3, 3, 3]
    assert get_option(groups[0], b"num_chunks") == -1 and get_option(groups[0], b"force_kernel_less") == 0
    set_option(groups[0], b"num_chunks", 6)
    set_option(groups[1], b"force_kernel_less", 1)
    assert get_option(groups[0], b"num_chunks") == 6 and get_option(groups[1], b"num_chunks") == -1
    assert get_option(groups[1], b"force_kernel_less") == 1
    assert get_pkl(groups[2]) is False
    set_pkl(groups[2], True)
    assert get_pkl(groups[2]) is True and get_option(groups[2], b"prefer_kernel_less") == 1
    for g in groups:
        destroy(g)


def test_the_python_module_loaded_its_core_through_the_entry():
    from moodist_amd import _C

    info = _C.core_api_info()
    assert info["entry"] == "moodistGetApi" and info["version"] == API_VERSION and info["magic"] == build_magic()
    assert info["slots"] == 69 and os.path.samefile(info["path"], LIB)


def test_a_core_of_another_build_is_refused_by_its_magic(tmp_path):
    # The reference draws a build magic per configure so that a stale libmoodist.so beside a new
    # _C is caught (CMakeLists.txt:97-106; wrapper/moodist_loader.cc:363-386).  Here: a Python
    # module built with another magic, placed beside the built core, must refuse to load it.
    import shutil
    import subprocess
    import sys
    import sysconfig

    suffix = sysconfig.get_config_var("EXT_SUFFIX")
    other = tmp_path / ("_C" + suffix)
    env = dict(os.environ, MOODIST_BUILD_MAGIC="0x0123456789abcdefULL")
    subprocess.run([sys.executable, os.path.join(ROOT, "moodist_amd", "csrc", "wrapper", "build_wrapper.py"), str(other)],
                   check=True, capture_output=True, text=True, env=env)
    shutil.copy(LIB, tmp_path / "libmoodist.so")
    code = ("import importlib.util, sys\n"
            "spec = importlib.util.spec_from_file_location('_C', %r)\n"
            "m = importlib.util.module_from_spec(spec)\n"
            "spec.loader.exec_module(m)\n" % str(other))
    r = subprocess.run([sys.executable, "-c", "import torch\n" + code], capture_output=True, text=True, timeout=300)
    assert r.returncode != 0
    assert "build magic mismatch" in r.stderr, r.stderr[-2000:]
    # and the module of THIS build loads the same copy of the core
    mine = tmp_path / "same" / ("_C" + suffix)
    os.makedirs(mine.parent)
    shutil.copy(os.path.join(ROOT, "moodist_amd", "_C" + suffix), mine)
    shutil.copy(LIB, mine.parent / "libmoodist.so")
    r = subprocess.run([sys.executable, "-c", "import torch\n" + code.replace(str(other), str(mine)) +
                        "print(m.core_api_info()['magic'])\n"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert int(r.stdout.strip()) == build_magic()
