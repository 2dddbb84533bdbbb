"""The boundary as files: include/compat mirrors the reference's include paths with one-line forwarders, and
include/fitre_blas_compat.h spells the vendor BLAS names as macros over the C-ABI.  Checked here: a caller written with the
reference's paths and names compiles with -Werror and links; and, where the reference tree is present, its own unchanged
sources on either side of the boundary parse against these headers (nothing of the reference is copied or run: the compiler
only reads it)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INC = ["-I", os.path.join(ROOT, "include", "compat"), "-I", os.path.join(ROOT, "include")]
REFERENCE = "/root/reference"


def test_caller_with_the_reference_spelling_compiles_and_links(tmp_path):
    exe = str(tmp_path / "compat_caller")
    lib_dir = os.path.join(ROOT, "fitre_amd")
    build = subprocess.run(["gcc", "-std=c11", "-Wall", "-Wextra", "-Werror"] + INC +
                           [os.path.join(ROOT, "tests", "c_api", "compat_caller.c"), "-o", exe, "-L", lib_dir, "-lfitre_cnn",
                            "-lfitre_hip", "-lm", "-Wl,-rpath," + lib_dir], capture_output=True, text=True)
    assert build.returncode == 0, build.stderr
    assert subprocess.run([exe]).returncode == 0


def test_every_forwarder_includes_cleanly(tmp_path):
    compat = os.path.join(ROOT, "include", "compat")
    names = sorted(os.path.join(d, f)[len(compat) + 1:] for d, _, fs in os.walk(compat) for f in fs)
    assert len(names) >= 35
    src = tmp_path / "all.c"
    src.write_text("".join("#include <%s>\n" % n for n in names) + "int main(void) { return 0; }\n")
    for compiler, std in (("gcc", "-std=c11"), ("g++", "-std=c++11")):
        out = subprocess.run([compiler, std, "-Wall", "-Werror", "-fsyntax-only", "-x", "c" if compiler == "gcc" else "c++"] + INC +
                             [str(src)], capture_output=True, text=True)
        assert out.returncode == 0, out.stderr


# unchanged reference sources: a solver (the FC family's caller), the KFAC bookkeeping, and the reference's own
# computeCNNGradient / evaluateCNNModel bodies, which call cnnForward / cnnBackward across the boundary
REFERENCE_CALLERS = [("solvers/cg_steihaug.c", "c"), ("solvers/kfac_utils.cu", "c++"), ("functions/cnn_gradient.cu", "c++"),
                     ("functions/cnn_eval_model.cu", "c++")]


@pytest.mark.skipif(not os.path.isdir(REFERENCE), reason="the reference tree is not on this machine")
@pytest.mark.parametrize("path,lang", REFERENCE_CALLERS)
def test_unchanged_reference_source_parses_against_the_headers(path, lang):
    compiler = ["gcc", "-std=gnu99"] if lang == "c" else ["g++", "-std=c++11", "-fpermissive"]
    out = subprocess.run(compiler + ["-fsyntax-only", "-x", lang] + INC + ["-I", REFERENCE, os.path.join(REFERENCE, path)],
                         capture_output=True, text=True)
    assert out.returncode == 0 and "error" not in out.stderr, out.stderr
