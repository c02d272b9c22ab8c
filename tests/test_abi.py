"""The C-ABI library loads on a machine without a GPU and exports every entry point include/crit_pkv.h declares; the
Python mirror of the parameter structs has the library's sizes. No compute call is made here."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "crit_pkv.h")


def _declared():
    text = open(HEADER, encoding="utf-8").read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(crit_pkv_\w+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    from crit_amd.paged_kv_attention import _abi
    return _abi.load()


def test_the_header_declares_the_entry_points():
    names = _declared()
    for want in ("crit_pkv_write", "crit_pkv_attend", "crit_pkv_merge", "crit_pkv_prefill", "crit_pkv_error",
                 "crit_pkv_params_size", "crit_pkv_abi_version", "crit_pkv_stream_read"):
        assert want in names


def test_the_header_is_plain_c(tmp_path):
    # what a cgo / JNI / ctypes binding includes: C99, pedantic, no warning; and the same text as C++
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    source = tmp_path / "use.c"
    source.write_text('#include "crit_pkv.h"\nint main(void) { crit_pkv_attend_params p; (void)p; return CRIT_PKV_ABI_VERSION > 0 ? 0 : 1; }\n')
    include = os.path.join(ROOT, "include")
    for command in (["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror"], ["g++", "-std=c++17", "-Wall", "-Werror", "-x", "c++"]):
        done = subprocess.run(command + ["-I", include, "-fsyntax-only", str(source)], capture_output=True, text=True)
        assert done.returncode == 0, done.stderr


def test_a_c_program_links_the_library_and_is_refused_a_null_launch(tmp_path, lib):
    # the boundary as a cgo / JNI stub meets it: a C99 program, the header, the shared library; no GPU is touched (the
    # launch is refused for its NULL pointers before any HIP call)
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    from crit_amd.paged_kv_attention import _abi
    library = next(path for path in _abi.candidates() if os.path.exists(path))
    source = tmp_path / "use.c"
    source.write_text("""#include <stdio.h>
#include <string.h>
#include "crit_pkv.h"
int main(void) {
    crit_pkv_attend_params p;
    memset(&p, 0, sizeof p);
    if (crit_pkv_abi_version() != CRIT_PKV_ABI_VERSION) return 2;
    int code = crit_pkv_attend(&p, NULL);
    printf("%d %s", code, crit_pkv_error(code));
    return code == CRIT_PKV_E_NULL ? 0 : 3;
}
""")
    where = os.path.dirname(library)
    program = tmp_path / "use"
    built = subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(source), "-o", str(program),
                            "-L", where, "-lcrit_pkv", f"-Wl,-rpath,{where}", "-Wl,-rpath,/opt/rocm/lib"], capture_output=True, text=True)
    assert built.returncode == 0, built.stderr
    ran = subprocess.run([str(program)], capture_output=True, text=True, timeout=60)
    assert ran.returncode == 0 and "NULL" in ran.stdout, (ran.returncode, ran.stdout, ran.stderr)


def test_the_library_exports_every_declared_symbol(lib):
    for name in _declared():
        assert hasattr(lib, name), name


def test_struct_mirrors_match_the_library(lib):
    from crit_amd.paged_kv_attention import _abi
    assert lib.crit_pkv_abi_version() == _abi.ABI_VERSION
    for which, struct in enumerate((_abi.WriteParams, _abi.AttendParams, _abi.MergeParams, _abi.PrefillParams)):
        assert lib.crit_pkv_params_size(which) == ctypes.sizeof(struct)
    assert lib.crit_pkv_params_size(99) == -1


def test_error_strings(lib):
    assert lib.crit_pkv_error(0) == b"ok"
    for code in (-1, -2, -3, -4):
        assert lib.crit_pkv_error(code).startswith(b"crit_pkv:")
    from crit_amd.paged_kv_attention import _abi
    with pytest.raises(ValueError, match="crit_pkv"):
        _abi.check(-1, "x")
    _abi.check(0, "x")


def test_null_parameters_are_refused_without_touching_a_gpu(lib):
    from crit_amd.paged_kv_attention import _abi
    for fn, struct in ((lib.crit_pkv_write, _abi.WriteParams), (lib.crit_pkv_attend, _abi.AttendParams),
                       (lib.crit_pkv_merge, _abi.MergeParams), (lib.crit_pkv_prefill, _abi.PrefillParams)):
        assert fn(ctypes.byref(struct()), None) == -3          # CRIT_PKV_E_NULL: nothing was launched


def test_the_module_keeps_the_reference_interface():
    # names and signatures crit's KVPool and DeviceAttention call (reference __init__.py:74-80, 260-362, 396-400, 1245)
    import inspect
    import crit_amd.paged_kv_attention as pk
    assert pk.MAX_COLUMNS == 64 and pk.KINDS == {"bf16": 0, "fp16": 0, "fp8": 1, "fp8:row": 2, "int8": 3}
    for name in ("write", "attend", "prefill", "partitions", "piece_size", "tile_for", "workspace_floats", "flash_chunk",
                 "flash_parts", "flash_block", "flash_tile", "cuda_chunk", "cuda_parts", "cuda_prompt", "owner", "release"):
        assert callable(getattr(pk, name)), name
    write = inspect.signature(pk.write).parameters
    assert list(write)[:9] == [
        "keys", "values", "slots", "key_pages", "value_pages", "kind", "key_scales", "value_scales", "multipliers"]
    # (beyond the reference's: the keys' rotary embedding, and their RMS norm in front of it, fused into the append, by
    # keyword only)
    assert list(write)[9:] == ["rope", "norm"]
    for extra in ("rope", "norm"):
        assert write[extra].kind is inspect.Parameter.KEYWORD_ONLY and write[extra].default is None
    attend = inspect.signature(pk.attend).parameters
    assert list(attend)[:10] == ["q", "key_pages", "value_pages", "kind", "tables", "rows", "starts", "firsts", "columns",
                                 "page"]
    for name in ("counts", "offsets", "tokens", "key_scales", "value_scales", "multipliers", "scale", "partitions",
                 "parents", "blocks", "block_size", "out", "lse", "workspace", "piece", "fused", "fresh", "flash", "chunk",
                 "sinks", "sliding", "derive"):
        assert attend[name].kind is inspect.Parameter.KEYWORD_ONLY, name
    prefill = inspect.signature(pk.prefill).parameters
    assert list(prefill)[:7] == ["q", "key_pages", "value_pages", "kind", "table", "position", "page"]
    assert pk.workspace_floats(3, 8, 16, 128) == 3 * 8 * 16 * 130
    assert pk.tile_for(1, 4, (9, 5))[0] // 4 == 1 and pk.tile_for(5, 4, (9, 5))[0] // 4 <= 5
    assert pk.piece_size(128, 128, "bf16") % 16 == 0 and pk.flash_chunk(128, 128, 32, 8, 16) % pk.flash_block(128, 128, 32, 8, 16) == 0
    assert pk.flash_parts(200_000, 1024) == 196 and pk.cuda_prompt(128, 128, None, "bf16", "cuda") is False
    with pk.owner("a"):
        pass
    pk.release("a")


def test_the_pool_functions_refuse_host_tensors_and_bad_shapes_before_any_launch():
    # (host logic only: every check below fails before a kernel could be launched, so it runs without a GPU)
    import pytest
    import torch
    import crit_amd.paged_kv_attention as pk
    tables = torch.zeros(2, 4, dtype=torch.int32)
    capacity = torch.zeros(2, dtype=torch.int64)
    i64 = torch.zeros(3, dtype=torch.int64)
    with pytest.raises(ValueError, match="GPU"):
        pk.slots_at(tables, capacity, i64, i64, 16, 8)
    with pytest.raises(ValueError, match="GPU"):
        pk.compact([torch.zeros(1, 8, 2, 16)], 8, tables, capacity, i64, i64, torch.zeros(1, 4, dtype=torch.int64), i64, 16, 8)
    with pytest.raises(ValueError):
        pk.copy_pages([], 8, i64, i64, 4)
    with pytest.raises(ValueError, match="GPU"):
        pk.copy_pages([torch.zeros(1, 8, 2, 16)], 8, i64, i64, 4)
    with pytest.raises(ValueError):
        pk.rows_at(torch.zeros(8, 2, 16, dtype=torch.bfloat16), None, "bf16", i64.to(torch.int32))
    with pytest.raises(ValueError, match="GPU"):
        pk.rows_at(torch.zeros(8, 2, 16, dtype=torch.bfloat16), None, "bf16", i64)
    with pytest.raises(ValueError):
        pk.gather(torch.zeros(8, 2, 16, dtype=torch.bfloat16), None, "bf16", torch.zeros(1, dtype=torch.int32), 40, 16)
    with pytest.raises(ValueError, match="rope rotates keys"):
        pk.write(None, torch.zeros(1, 2, 16), i64[:1], None, torch.zeros(8, 2, 16), "bf16", rope=(None, None))
