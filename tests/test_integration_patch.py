"""The engine integration as artifacts: integration/leelaz-use-hip.patch applies to the
reference's own sources, and both drop-in classes (lzhip::HIPScheduler from
include/forward_pipe.h, the C-ABI adapter integration/HIPPipeAdapter.h) compile against the
engine's real ForwardPipe.h / Network.h, so that every `override` is checked against the
reference's signatures (src/ForwardPipe.h:38-71, src/Network.h:66-67).  Compile checks are
syntax-only: the engine's other translation units need Boost, which this image lacks.
Skipped where the reference tree is absent."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference"
PATCH = os.path.join(ROOT, "integration", "leelaz-use-hip.patch")
PATCHED = ["CMakeLists.txt", "src/Network.cpp", "src/Network.h", "src/UCTSearch.cpp"]

need_ref = pytest.mark.skipif(not os.path.isdir(os.path.join(REF, "src")) or shutil.which("g++") is None,
                              reason="needs the reference tree and g++")


def syntax_only(args, src):
    cmd = ["g++", "-std=c++14", "-fsyntax-only", "-Wall", "-Wextra"] + args + [src]
    return subprocess.run(cmd, capture_output=True, text=True)


@need_ref
def test_drop_in_classes_compile_against_the_engine_headers():
    r = syntax_only(["-DUSE_CPU_ONLY", "-DLZHIP_ENGINE_BUILD", "-I", os.path.join(REF, "src"),
                     "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "integration")],
                    os.path.join(ROOT, "tests", "cpp", "engine_adapter_check.cpp"))
    assert r.returncode == 0, r.stderr


@need_ref
@pytest.mark.skipif(shutil.which("patch") is None, reason="needs patch")
def test_patch_applies_and_the_patched_header_compiles_in_hip_mode(tmp_path):
    for f in PATCHED:
        dst = tmp_path / f
        dst.parent.mkdir(parents=True, exist_ok=True)
        shutil.copy(os.path.join(REF, f), dst)
    r = subprocess.run(["patch", "-p1", "--no-backup-if-mismatch", "-i", PATCH], cwd=tmp_path,
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "FAILED" not in r.stdout and "fuzz" not in r.stdout, r.stdout
    net = (tmp_path / "src" / "Network.cpp").read_text()
    assert "std::make_unique<lzhip::HIPScheduler>" in net and '#include "forward_pipe.h"' in net
    cm = (tmp_path / "CMakeLists.txt").read_text()
    assert "option(USE_HIP" in cm and "target_link_libraries(leelaz lzhip)" in cm
    # the engine's run-time self-check against CPUPipe stays compiled in (config.h is not
    # touched), and the search prints the library's batch counters where it printed OpenCL's
    uct = (tmp_path / "src" / "UCTSearch.cpp").read_text()
    assert "lzhip::batch_stats.single_evals" in uct and '#include "forward_pipe.h"' in uct
    # the patched Network.h with USE_HIP on (USE_OPENCL, USE_HALF and the self-check stay
    # defined, no OpenCL header is pulled in) together with the library's header
    tu = tmp_path / "hip_mode.cpp"
    tu.write_text('#include "config.h"\n#include "Network.h"\n#include "forward_pipe.h"\n'
                  "#if !defined(USE_OPENCL) || !defined(USE_HALF) || !defined(USE_OPENCL_SELFCHECK)\n"
                  '#error "unexpected switches in a USE_HIP build"\n#endif\n'
                  "int main() { lzhip::HIPScheduler s(LZHIP_FP16, 8, 0); ForwardPipe* p = &s; "
                  "return p == nullptr || lzhip::batch_stats.batch_evals.load() != 0; }\n")
    r = syntax_only(["-DUSE_HIP", "-DLZHIP_ENGINE_BUILD", "-I", str(tmp_path / "src"),
                     "-I", os.path.join(REF, "src"), "-I", os.path.join(ROOT, "include")], str(tu))
    assert r.returncode == 0, r.stderr
