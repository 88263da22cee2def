"""The Rust binding sources kept in-tree (bitnet-mlx.rs_amd/rust/bitnet-hip) cannot be compiled here (no Rust
toolchain), so their extern "C" block is checked against include/bitnet_hip.h textually: same symbols, same
argument counts, same parameter names in the same order, same status constants."""
import re
from pathlib import Path

import bitnet_hip as bh

ROOT = Path(__file__).resolve().parents[1]
FFI = ROOT / "bitnet-mlx.rs_amd" / "rust" / "bitnet-hip" / "src" / "ffi.rs"


def header_prototypes():
    text = re.sub(r"/\*.*?\*/", "", bh.HEADER_PATH.read_text(), flags=re.S)
    protos = {}
    for m in re.finditer(r"\b(bitnet_hip_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        args = [a.strip() for a in m.group(2).split(",")]
        if args == ["void"]:
            args = []
        names = [re.sub(r"\[.*\]", "", a).split()[-1].lstrip("*") for a in args]
        protos[m.group(1)] = names
    return protos, text


def rust_prototypes():
    text = FFI.read_text()
    protos = {}
    for m in re.finditer(r"pub fn (bitnet_hip_[a-z0-9_]+)\s*\((.*?)\)\s*(?:->[^;]*)?;", text, flags=re.S):
        args = [a.strip() for a in m.group(2).split(",") if a.strip()]
        protos[m.group(1)] = [a.split(":")[0].strip() for a in args]
    return protos, text


def test_rust_extern_block_matches_header():
    c_protos, c_text = header_prototypes()
    r_protos, r_text = rust_prototypes()
    assert set(r_protos) == set(c_protos)
    for name, c_args in c_protos.items():
        assert r_protos[name] == c_args, name
    c_consts = dict(re.findall(r"(BITNET_HIP_[A-Z0-9_]+)\s*=\s*(\d+)", c_text)) | dict(
        re.findall(r"#define\s+(BITNET_HIP_[A-Z0-9_]+)\s+(\d+)", c_text))
    r_consts = dict(re.findall(r"pub const (BITNET_HIP_[A-Z0-9_]+): c_int = (\d+);", r_text))
    for name, value in r_consts.items():
        assert c_consts.get(name) == value, name
    assert {k for k in c_consts if not k.startswith("BITNET_HIP_PROJ_")} <= set(r_consts)


def test_rust_build_script_compiles_the_same_sources_with_the_same_flags():
    build_rs = (FFI.parents[1] / "build.rs").read_text()
    makefile = (ROOT / "bitnet-mlx.rs_amd" / "Makefile").read_text()
    for src in re.findall(r"csrc/([a-z0-9_]+\.hip)", makefile):
        assert f'"{src}"' in build_rs, src
    for flag in ("--offload-arch=gfx950", "-ffp-contract=off", "-fhip-fp32-correctly-rounded-divide-sqrt", "-packed-fp32-ops",
                 "-amdgpu-kernarg-preload-count=10"):
        assert flag in build_rs and flag.lstrip("-") in makefile.replace("$(ARCH)", "gfx950")
