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
    make_srcs = re.findall(r"csrc/([a-z0-9_]+\.hip)", re.search(r"^SRCS\s*=(.*)$", makefile, flags=re.M).group(1))
    decl = re.search(r"const KERNELS:\s*([^=]+?)\s*=\s*&?\[(.*?)\];", build_rs, flags=re.S)
    assert decl, "build.rs declares no KERNELS list"
    listed = re.findall(r'"([a-z0-9_]+\.hip)"', decl.group(2))
    assert listed == make_srcs  # the same sources in the same order as the Makefile's SRCS
    fixed_len = re.fullmatch(r"\[&str;\s*(\d+)\]", decl.group(1))
    if fixed_len:  # a fixed-size array type must state the number of elements it holds (a mismatch does not compile)
        assert int(fixed_len.group(1)) == len(listed)
    else:
        assert decl.group(1) == "&[&str]"
    for src in listed:
        assert (ROOT / "bitnet-mlx.rs_amd" / "csrc" / src).is_file(), src
    for flag in ("--offload-arch=gfx950", "-ffp-contract=off", "-fhip-fp32-correctly-rounded-divide-sqrt", "-packed-fp32-ops",
                 "-amdgpu-kernarg-preload-count=10"):
        assert flag in build_rs and flag.lstrip("-") in makefile.replace("$(ARCH)", "gfx950")


def _trait_methods(text, header_regex):
    """{method: [argument names]} of the trait / impl block that starts at header_regex (brace matched)."""
    m = re.search(header_regex, text)
    assert m, header_regex
    i = text.index("{", m.end() - 1)
    depth, j = 0, i
    while True:
        depth += text[j] == "{"
        depth -= text[j] == "}"
        if depth == 0:
            break
        j += 1
    body = re.sub(r"//[^\n]*", "", text[i:j])
    out = {}
    for fm in re.finditer(r"\bfn\s+([a-z_0-9]+)\s*\(([^)]*)\)", body, flags=re.S):
        args = [a.strip() for a in fm.group(2).split(",") if a.strip()]
        out[fm.group(1)] = [a if a.startswith("&") else a.split(":")[0].strip() for a in args]
    return out


def test_rust_crate_implements_the_reference_traits():
    """impl BitLinearForward / TernaryLookupKernel / I2SLookupKernel / InferenceBackend for the wrapper types: same
    method names, same receivers, same argument names and counts as the traits of the reference (transcribed with
    their file:line into tests/golden; compared with the reference's own text where that is present)."""
    import json

    traits = json.loads((ROOT / "tests" / "golden" / "reference_vectors.json").read_text())["rust_traits"]
    lib = (FFI.parent / "lib.rs").read_text()
    for trait, spec in traits.items():
        got = _trait_methods(lib, rf"impl\s+{trait}\s+for\s+{spec['for']}\s*\{{")
        assert got == spec["methods"], (trait, got)
        ref_file = Path("/root/reference") / spec["source"].split(":")[0]
        if ref_file.exists():
            assert _trait_methods(ref_file.read_text(), rf"pub\s+trait\s+{trait}\b[^{{]*\{{") == spec["methods"], trait


def test_rust_crate_gates_the_library_behind_its_feature_and_keeps_raw_pointers_unsafe():
    ffi = FFI.read_text()
    assert re.search(r'#\[cfg\(feature = "hip"\)\]\s*extern "C" \{', ffi)
    lib = (FFI.parent / "lib.rs").read_text()
    # every function that takes raw device pointers is an unsafe fn; DeviceTensor's fields are private
    for m in re.finditer(r"pub (unsafe )?fn ([a-z_0-9]+)\s*\(([^)]*)\)", lib, flags=re.S):
        if "*const" in m.group(3) or "*mut" in m.group(3):
            assert m.group(1), m.group(2)
    tensor = re.search(r"pub struct DeviceTensor \{(.*?)\}", lib, flags=re.S).group(1)
    assert "pub " not in tensor
    assert "HipNotEnabled" in lib and '#[cfg(not(feature = "hip"))]' in lib


def test_rust_quantizer_wrappers_call_the_library_and_use_the_model():
    """The safe layer reaches the quantiser entry points (not only declares them), implements the reference's Quantizer
    trait (quantization/mod.rs:96-116: quantize, dequantize, config, validate_input, get_stats) for the weight pipeline and
    the dynamic activation quantiser, and optimize_model builds its decoder from the Model it is given."""
    lib = (FFI.parent / "lib.rs").read_text()
    for sym in ("bitnet_hip_absmax_quantize_activations", "bitnet_hip_quantize_weights_reference", "bitnet_hip_abs_max",
                "bitnet_hip_quantize_activations_scaled", "bitnet_hip_bitlinear_set_weights_gguf", "bitnet_hip_decoder_set_chains"):
        assert f"ffi::{sym}(" in lib, sym
    for target in ("HipBitNetWeightQuantizer", "HipActivationQuantizerAdapter"):
        methods = _trait_methods(lib, rf"impl Quantizer for {target}\s*\{{")
        assert set(methods) == {"quantize", "dequantize", "config", "validate_input", "get_stats"}, target
        assert methods["quantize"][0] == "&self" and len(methods["quantize"]) == 2
    body = lib[lib.index("fn optimize_model(&mut self, model: &Model)"):]
    body = body[:body.index("fn get_memory_usage")]
    assert "decoder_shape_of(model)" in body and "let _ = model" not in body and "bind_decoder" in body
    assert "model.architecture" in lib
    # the state machine of DynamicActivationQuantizer, as the reference writes it (activations.rs:252-257)
    assert "self.config.ema_decay * prev + (1.0 - self.config.ema_decay) * current_scale" in lib
