"""The drop-in boundary against the reference's own sources (CPU, needs the reference tree and clang).

  * The reference's callers of src/nn/fast_metal.h -- wmat.c, fast_sft.c, fast_grpo.c, fast_inference.c -- must
    compile against include/fast_hip.h put in that header's place: same names, argument counts and types at every
    call site.
  * llm_metal_amd/compat/fast_sft_compat.c (the constructors and the adapter sync with the reference's signatures)
    must compile against the reference's qwen3.h / gemma3.h, and a reference caller of fast_sft.h (fast_grpo.c,
    main.c) must compile with llm_metal_amd/compat/fast_sft_compat.h in that header's place.
  * llm_metal_amd/compat/fast_inference_compat.c (inference_state_create*, qwen3_generate_fast*) likewise, in the place
    of fast_inference.h / fast_inference.c.
  * llm_metal_amd/compat/metal_backend_off.c must define every function src/core/metal_backend.h declares, with
    that header's prototypes.
  * The whole reference tree (main.c and every src/**/*.c except fast_sft.c and fast_inference.c, which the library
    replaces) links against libllm_metal_hip.so and the compat units with no undefined symbol.
  * tests/compat_probe.c runs the compat units on models built by the reference's own constructors, with the library
    entry points replaced by doubles that compare every field of the model description (host only, no GPU).

The reference's sources are compiled where they lie; nothing of them is copied."""
import os
import re
import shutil
import subprocess

import pytest

import glob

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


def test_inference_compat_unit_compiles_against_the_reference_model_structs(tmp_path):
    obj = tmp_path / "fast_inference_compat.o"
    clang(["-c", "-O1", "-DFAST_METAL_H", "-I", os.path.join(REF, "src", "nn"), "-I", INC,
           os.path.join(COMPAT, "fast_inference_compat.c"), "-o", str(obj)])
    syms = subprocess.run(["nm", "--defined-only", str(obj)], capture_output=True, text=True).stdout
    for fn in ("inference_state_create", "inference_state_create_gemma3", "qwen3_generate_fast", "qwen3_generate_fast_batch"):
        assert re.search(rf"\bT {fn}\b", syms), fn


def test_compat_inference_header_declares_what_fast_inference_h_declares():
    """Every function of src/nn/fast_inference.h is declared, with the same parameter list, by fast_inference_compat.h or
    by include/inference_hip.h (which it includes)."""
    def protos(text):
        text = re.sub(r"/\*.*?\*/", " ", re.sub(r"//.*", "", text), flags=re.S)
        out = {}
        for m in re.finditer(r"([A-Za-z_][\w \*]*?)\b(\w+)\s*\(([^;{}()]*)\)\s*;", text):
            params = [re.sub(r"\s+", " ", re.sub(r"\b\w+$", "", p.strip())).strip() for p in m.group(3).split(",")]
            out[m.group(2)] = params
        return out
    ref = protos(open(os.path.join(REF, "src", "nn", "fast_inference.h")).read())
    ours = protos(open(os.path.join(COMPAT, "fast_inference_compat.h")).read())
    ours.update(protos(open(os.path.join(INC, "inference_hip.h")).read()))
    assert len(ref) == 13, sorted(ref)
    for name, params in ref.items():
        assert name in ours, name
        assert [p.replace(" ", "") for p in ours[name]] == [p.replace(" ", "") for p in params], (name, ours[name], params)


REPLACED = ("fast_sft.c", "fast_inference.c")
LIB = os.path.join(ROOT, "llm_metal_amd", "libllm_metal_hip.so")


def reference_sources(dirs):
    out = []
    for d in dirs:
        out += sorted(f for f in glob.glob(os.path.join(REF, "src", d, "*.c")) if os.path.basename(f) not in REPLACED)
    return out


@pytest.mark.skipif(not os.path.exists(LIB), reason="libllm_metal_hip.so is not built")
def test_the_reference_tree_links_against_the_library(tmp_path):
    """./llm of the reference with fast_sft.c, fast_inference.c, fast_metal.m and metal_backend.m taken out and the
    library plus the compat units put in: the link line a maintainer of the reference would use.  No undefined symbol, and
    the binary starts."""
    exe = tmp_path / "llm_hip"
    r = subprocess.run([CLANG, "-std=c17", "-D_GNU_SOURCE", "-O1", "-w", "-DFAST_METAL_H",
                        "-include", os.path.join(COMPAT, "fast_inference_compat.h"), "-I", INC, "-I", os.path.join(REF, "src", "nn"),
                        "-I", os.path.join(REF, "src"), "-I", REF, os.path.join(REF, "main.c")] +
                       reference_sources(["core", "nn", "data", "train"]) +
                       [os.path.join(COMPAT, f) for f in ("fast_sft_compat.c", "fast_inference_compat.c", "metal_backend_off.c")] +
                       ["-L", os.path.dirname(LIB), "-lllm_metal_hip", "-Wl,-rpath," + os.path.dirname(LIB), "-Wl,--no-undefined",
                        "-lm", "-lpthread", "-o", str(exe)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-4000:]
    undefined = subprocess.run(["nm", "-u", str(exe)], capture_output=True, text=True).stdout
    ours = [l.split()[-1] for l in undefined.splitlines() if re.search(r"\b(metal_|sft_|inference_|wmat_|hip_|fast_metal_|grpo_)", l)]
    exported = subprocess.run(["nm", "-D", "--defined-only", LIB], capture_output=True, text=True).stdout
    for sym in ours:
        assert re.search(rf"\bT {re.escape(sym)}\b", exported), sym        # every one of them is the library's
    assert len(ours) >= 40, len(ours)
    out = subprocess.run([str(exe), "--help"], capture_output=True, text=True, timeout=60)
    assert "--mode sft" in out.stdout + out.stderr


def test_compat_units_map_the_reference_model_structs(tmp_path):
    exe = tmp_path / "compat_probe"
    srcs = [f for f in reference_sources(["core", "nn", "data"]) if os.path.basename(f) not in ("fast_grpo.c", "wmat.c")]
    r = subprocess.run([CLANG, "-std=c17", "-D_GNU_SOURCE", "-O1", "-w", "-DFAST_METAL_H", "-I", COMPAT, "-I", INC,
                        "-I", os.path.join(REF, "src", "nn"), "-I", os.path.join(REF, "src"), "-I", REF,
                        os.path.join(ROOT, "tests", "compat_probe.c")] + srcs +
                       [os.path.join(COMPAT, f) for f in ("fast_sft_compat.c", "fast_inference_compat.c", "metal_backend_off.c")] +
                       ["-lm", "-lpthread", "-o", str(exe)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-4000:]
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    fails = [l for l in run.stdout.splitlines() if l.startswith("FAIL")]
    assert run.returncode == 0 and not fails, (fails[:10], run.stderr[-2000:])
    assert run.stdout.count("\nok ") > 400 and "PASSED" in run.stdout
    # adapters of another rank are refused with a message, not silently
    assert "attached adapters are ignored" in run.stderr
