"""The drop-in boundary against the reference's own sources (CPU, needs the reference tree and clang).

  * The reference's callers of src/nn/fast_metal.h -- wmat.c, fast_sft.c, fast_grpo.c, fast_inference.c -- must
    compile against include/fast_hip.h put in that header's place: same names, argument counts and types at every
    call site.
  * llm_metal_amd/compat/fast_sft_compat.c (the constructors and the adapter sync with the reference's signatures)
    must compile against the reference's qwen3.h / gemma3.h, and a reference caller of fast_sft.h (fast_grpo.c,
    main.c) must compile with llm_metal_amd/compat/fast_sft_compat.h in that header's place.
  * llm_metal_amd/compat/metal_backend_off.c must define every function src/core/metal_backend.h declares, with
    that header's prototypes.

Nothing of the reference is linked or run: these are compile checks of the interface."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference"
INC = os.path.join(ROOT, "include")
COMPAT = os.path.join(ROOT, "llm_metal_amd", "compat")
CLANG = shutil.which("clang") or "/opt/rocm/lib/llvm/bin/clang"

pytestmark = pytest.mark.skipif(not os.path.isdir(os.path.join(REF, "src", "nn")) or not os.path.exists(CLANG),
                                reason="needs the reference tree and clang")
BASE = [CLANG, "-std=c17", "-D_GNU_SOURCE", "-Wall", "-Werror=implicit-function-declaration", "-Werror=incompatible-pointer-types",
        "-Werror=int-conversion", "-Wno-unused", "-Wno-unknown-pragmas"]


def clang(args, **kw):
    r = subprocess.run(BASE + args, capture_output=True, text=True, **kw)
    assert r.returncode == 0, r.stderr[-4000:]
    return r


@pytest.mark.parametrize("src", ["wmat.c", "fast_sft.c", "fast_grpo.c", "fast_inference.c"])
def test_reference_callers_compile_against_fast_hip_h(src):
    clang(["-fsyntax-only", "-include", os.path.join(INC, "fast_hip.h"), "-DFAST_METAL_H",
           "-I", os.path.join(REF, "src", "nn"), os.path.join(REF, "src", "nn", src)])


def test_compat_adapters_compile_against_the_reference_model_structs(tmp_path):
    obj = tmp_path / "fast_sft_compat.o"
    clang(["-c", "-O1", "-DFAST_METAL_H", "-I", os.path.join(REF, "src", "nn"), "-I", INC,
           os.path.join(COMPAT, "fast_sft_compat.c"), "-o", str(obj)])
    syms = subprocess.run(["nm", "--defined-only", str(obj)], capture_output=True, text=True).stdout
    for fn in ("sft_state_create", "sft_state_create_gemma3", "sft_state_create_full", "sft_state_create_gemma3_full",
               "sft_sync_lora_to_model", "sft_sync_lora_to_gemma3"):
        assert re.search(rf"\bT {fn}\b", syms), fn


@pytest.mark.parametrize("src", ["src/nn/fast_grpo.c", "main.c"])
def test_reference_callers_of_fast_sft_h_compile_against_the_compat_header(src):
    """fast_grpo.c drives the GRPO route through the accessors; main.c's run_sft is the SFT driver
    (sft_state_create*, sft_train_step, sft_sync_lora_to_*, sft_save_*)."""
    clang(["-fsyntax-only", "-include", os.path.join(COMPAT, "fast_sft_compat.h"), "-DFAST_METAL_H",
           "-I", os.path.join(REF, "src", "nn"), "-I", os.path.join(REF, "src"), "-I", REF, "-I", INC,
           os.path.join(REF, src)])


def test_backend_off_unit_defines_every_legacy_symbol(tmp_path):
    obj = tmp_path / "metal_backend_off.o"
    clang(["-c", "-O1", "-I", os.path.join(REF, "src"), os.path.join(COMPAT, "metal_backend_off.c"), "-o", str(obj)])
    syms = subprocess.run(["nm", "--defined-only", str(obj)], capture_output=True, text=True).stdout
    defined = set(re.findall(r"\bT (\w+)", syms))
    text = re.sub(r"//.*", "", open(os.path.join(REF, "src", "core", "metal_backend.h")).read())
    declared = set(re.findall(r"\b(metal_\w+)\s*\(", text))
    assert len(declared) == 30
    assert declared == defined, (declared - defined, defined - declared)
