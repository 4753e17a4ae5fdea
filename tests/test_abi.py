"""The C ABI boundary on a host without a GPU: the library loads, exports exactly what
include/mxp.h declares, and reports errors through status codes (no compute here)."""

import ctypes as C
import json
import re
import struct
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


def _declared(header="mxp.h"):
    text = (ROOT / "include" / header).read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mxp_[a-z0-9_]+)\s*\(", text)))


BENCH_ONLY = ["mxp_describe_views", "mxp_engine_launch_times", "mxp_engine_set_launch_timing", "mxp_measure_gather", "mxp_measure_h2d",
              "mxp_measure_read", "mxp_set_transpose_form", "mxp_synth_device", "mxp_synth_host"]


def test_library_exports_every_declared_symbol(mxp):
    declared, bench = _declared(), _declared("mxp_bench.h")
    assert len(declared) >= 35
    # measurement and test-input entry points stay out of the drop-in header
    assert bench == BENCH_ONLY and not set(bench) & set(declared)
    out = subprocess.run(["nm", "-D", "--defined-only", str(mxp.LIB_PATH)], capture_output=True, text=True, check=True)
    exported = {line.split()[-1] for line in out.stdout.splitlines() if " T " in line}
    assert [s for s in declared + bench if s not in exported] == []
    # and nothing undeclared leaks out under the mxp_ prefix
    assert sorted(s for s in exported if s.startswith("mxp_")) == sorted(declared + bench)
    # the ctypes binding covers the same sets
    assert sorted(mxp.SIGNATURES) == declared and sorted(mxp.BENCH_SIGNATURES) == bench
    assert mxp.lib().mxp_abi_version() == 1


def test_rust_sys_generator_covers_the_header():
    """include/gen_rust_sys.py (no Rust toolchain here, so the output is checked for coverage and
    shape, not compiled): one ``pub fn`` per declared function with the same parameter count,
    one ``#[repr(C)]`` struct per typedef with the same field count, every MXP_* constant."""
    import importlib.util
    import re

    spec = importlib.util.spec_from_file_location("gen_rust_sys", ROOT / "include" / "gen_rust_sys.py")
    gen = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(gen)
    header = (ROOT / "include" / "mxp.h").read_text()
    out = gen.generate(header)
    consts, opaque, structs, funcs = gen.parse(header)
    assert sorted(name for _r, name, _p in funcs) == _declared()
    for ret, name, params in funcs:
        m = re.search(rf"pub fn {name}\((.*?)\)( -> [^;]+)?;", out)
        assert m, name
        assert (m.group(1).count(":") == len(params)) and (bool(m.group(2)) == (ret != "void")), name
    for sname, fields in structs.items():
        body = re.search(rf"pub struct {sname} \{{(.*?)\n\}}", out, flags=re.S).group(1)
        assert body.count("pub ") == len(fields), sname
    for o in opaque:
        assert f"pub struct {o} {{ _private: [u8; 0] }}" in out
    for name, _v in consts:
        assert f"pub const {name}:" in out
    assert "pub fn mxp_execute(engine: *mut mxp_engine, plan: *mut mxp_plan, dst_ptrs: *const *mut c_void, " \
           "stats: *mut mxp_exec_stats) -> c_int;" in out
    assert "pub shape: [i64; MXP_MAX_DIMS as usize]," in out and "pub const MXP_ERR_IO: i32 = -1;" in out


def test_header_is_plain_c(tmp_path):
    src = tmp_path / "t.c"
    src.write_text('#include "mxp.h"\n#include "mxp_bench.h"\nint main(void){ mxp_engine_options o; (void)o; return MXP_OK; }\n')
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", f"-I{ROOT / 'include'}", "-c", str(src), "-o",
                    str(tmp_path / "t.o")], check=True)


def test_struct_layouts_match_the_header(mxp, tmp_path):
    src = tmp_path / "s.c"
    src.write_text('#include <stdio.h>\n#include "mxp.h"\nint main(void){printf("%zu %zu %zu %zu %zu %zu %zu %zu\\n",'
                   "sizeof(mxp_tensor_info),sizeof(mxp_file_info),sizeof(mxp_write_info),sizeof(mxp_param_info),"
                   "sizeof(mxp_engine_options),sizeof(mxp_exec_stats),sizeof(mxp_box),sizeof(mxp_view_copy));return 0;}\n")
    exe = tmp_path / "s"
    subprocess.run(["gcc", f"-I{ROOT / 'include'}", str(src), "-o", str(exe)], check=True)
    sizes = [int(v) for v in subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.split()]
    assert sizes == [C.sizeof(mxp.TensorInfo), C.sizeof(mxp.FileInfo), C.sizeof(mxp.WriteInfo), C.sizeof(mxp.ParamInfo),
                     C.sizeof(mxp.EngineOptions), C.sizeof(mxp.ExecStats), C.sizeof(mxp.Box), C.sizeof(mxp.ViewCopy)]


def test_dtype_map_is_the_safetensors_one(mxp):
    lib = mxp.lib()
    for name, size in mxp.DTYPE_SIZE.items():  # gds_loader.py:36-49
        code = lib.mxp_dtype_from_name(name.encode())
        assert code == mxp.DTYPE_CODE[name] and lib.mxp_dtype_size(code) == size
        assert lib.mxp_dtype_name(code).decode() == name
    assert lib.mxp_dtype_from_name(b"F4") == -1 and lib.mxp_dtype_size(99) == 0


def _write(path, entries, blob, pad=0):
    body = json.dumps(entries).encode() + b" " * pad
    path.write_bytes(struct.pack("<Q", len(body)) + body + blob)


def test_checkpoint_error_classes(mxp, tmp_path):
    from modelexpress_amd.engine import Checkpoint

    def code(path):
        with pytest.raises(mxp.MxpError) as e:
            Checkpoint(str(path))
        return e.value.code, e.value.message

    assert code(tmp_path / "missing")[0] == mxp.ERR_IO
    short = tmp_path / "short.safetensors"
    short.write_bytes(b"\x00\x01")
    c, msg = code(short)
    assert c == mxp.ERR_FORMAT and "Invalid safetensors file" in msg  # gds_loader.py:254-255
    big = tmp_path / "big.safetensors"
    big.write_bytes(struct.pack("<Q", 100 * 1024 * 1024 + 1) + b"{}")
    c, msg = code(big)
    assert c == mxp.ERR_FORMAT and "header too large" in msg  # gds_loader.py:259-262
    trunc = tmp_path / "trunc.safetensors"
    trunc.write_bytes(struct.pack("<Q", 64) + b"{}")
    assert code(trunc)[0] == mxp.ERR_FORMAT
    bad = tmp_path / "bad.safetensors"
    _write(bad, {"x": {"dtype": "F4", "shape": [2], "data_offsets": [0, 1]}}, b"\0")
    c, msg = code(bad)
    assert c == mxp.ERR_UNSUPPORTED and "Unsupported safetensors dtype 'F4'" in msg  # gds_loader.py:305-309
    eof = tmp_path / "eof.safetensors"
    _write(eof, {"x": {"dtype": "U8", "shape": [8], "data_offsets": [0, 8]}}, b"abcd")
    assert code(eof)[0] == mxp.ERR_IO  # read past EOF, gds_transfer.py:182-186
    size = tmp_path / "size.safetensors"
    _write(size, {"x": {"dtype": "F32", "shape": [3], "data_offsets": [0, 8]}}, b"\0" * 8)
    assert code(size)[0] == mxp.ERR_FORMAT
    garbage = tmp_path / "garbage.safetensors"
    garbage.write_bytes(struct.pack("<Q", 5) + b"{nope")
    assert code(garbage)[0] == mxp.ERR_FORMAT
    empty_dir = tmp_path / "empty"
    empty_dir.mkdir()
    c, msg = code(empty_dir)
    assert c == mxp.ERR_IO and "No .safetensors files found" in msg
    (empty_dir / "model.safetensors.index.json").write_text('{"weight_map": {}}')
    c, msg = code(empty_dir)
    assert c == mxp.ERR_FORMAT and "Empty weight_map" in msg


def test_checkpoint_listing_matches_oracle(mxp, oracle, tmp_path):
    from modelexpress_amd import models, synth
    from modelexpress_amd.engine import Checkpoint

    layout = models.Llama(layers=1, hidden=32, ffn=64, q_heads=4, kv_heads=2, head_dim=8, vocab=64)
    synth.write_checkpoint(layout.checkpoint(), str(tmp_path), n_shards=3, seed=1)
    ck = Checkpoint(str(tmp_path))
    got = [(t.name, t.dtype, t.shape, t.file_offset, t.nbytes, ck.files()[t.file_index]["path"]) for t in ck.tensors()]
    want = []
    for path, names in oracle.resolve_safetensors_files(str(tmp_path)).items():
        info = oracle.parse_safetensors_header(path)
        for n in sorted(names, key=lambda n: info[n]["file_offset"]):
            want.append((n, info[n]["dtype"], tuple(info[n]["shape"]), info[n]["file_offset"], info[n]["size"], path))
    assert got == want
    assert ck.find("lm_head.weight") >= 0 and ck.find("nope") == -1


def test_plan_argument_errors(mxp, tmp_path):
    from modelexpress_amd import models, synth
    from modelexpress_amd.engine import Checkpoint, ParamSpec, PlacementPlan

    layout = models.Gpt2(layers=1, hidden=16, ffn=32, vocab=11, positions=4)
    synth.write_checkpoint(layout.checkpoint(), str(tmp_path), seed=1)
    ck = Checkpoint(str(tmp_path))
    with pytest.raises(mxp.MxpError) as e:
        PlacementPlan(ck, layout.rank_view().params, tp_size=2, tp_rank=2)
    assert e.value.code == mxp.ERR_ARG
    dup = [ParamSpec("a", "F16", (1,)), ParamSpec("a", "F16", (1,))]
    with pytest.raises(mxp.MxpError) as e:
        PlacementPlan(ck, dup, allow_unmapped=True, allow_uncovered=True)
    assert e.value.code == mxp.ERR_ARG
    plan = PlacementPlan(ck, layout.rank_view().params)
    assert plan.totals()["placed_bytes"] == sum(t.nbytes for t in layout.checkpoint())
    lib = mxp.lib()
    assert lib.mxp_plan_build(plan._h) == mxp.ERR_STATE  # already built
    assert lib.mxp_plan_add_skip_prefix(plan._h, b"x") == mxp.ERR_STATE
    assert lib.mxp_execute(None, plan._h, None, None) == mxp.ERR_ARG


def test_engine_create_without_a_gpu_is_an_error_not_a_crash(mxp):
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from modelexpress_amd.engine import PlacementEngine

    with pytest.raises(mxp.MxpError) as e:
        PlacementEngine(0)
    assert e.value.code == mxp.ERR_DEVICE


def test_missing_library_fails_loudly(mxp, monkeypatch, tmp_path):
    monkeypatch.setattr(mxp, "_lib", None)
    monkeypatch.setattr(mxp, "LIB_PATH", tmp_path / "libmxplace.so")
    with pytest.raises(mxp.MxpLibraryMissing, match="no fallback"):
        mxp.lib()
