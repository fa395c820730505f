"""The BVH builder's kernels compiled for the CPU (tests/cpu_build) and run under the address and undefined-behaviour
sanitizers on small scenes of every kind the GPU tests use: both ways of making the hierarchy (agglomeration, Morton
codes), both box fits, refits, the collapse to wide nodes, degenerate input (one point, identical quads, non-finite
corners), with the finished structure held against the invariants the walks rely on.  What is checked here cannot fault
a GPU later: every index the kernels form is formed here first."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)


def test_builder_kernels_on_the_cpu_under_sanitizers(tmp_path):
    exe = str(tmp_path / "builder_cpu")
    cmd = ["g++", "-std=c++20", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
           "-Wno-unknown-pragmas", "-Wno-attributes", "-I", os.path.join(HERE, "cpu_build"), "-I",
           os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "diff-surfel-tracing_amd", "csrc"), "-x", "c++",
           os.path.join(HERE, "cpu_build", "builder_cpu.cpp"), "-o", exe]
    subprocess.check_call(cmd)
    run = subprocess.run([exe], capture_output=True, text=True, timeout=900)
    if "ASan runtime does not come first" in run.stderr:
        # a library preloaded into every process keeps the sanitizer from starting: same run, structure checks only
        subprocess.check_call([c for c in cmd if not c.startswith("-fsanitize") and not c.startswith("-fno-sanitize")])
        run = subprocess.run([exe], capture_output=True, text=True, timeout=900)
    print(run.stdout[-4000:])
    assert run.returncode == 0, run.stdout[-2000:] + run.stderr[-4000:]
    assert "ALL OK" in run.stdout
    assert run.stdout.count(" agglomerated 1 ") >= 8 and "refused 1" not in run.stdout
