"""Host code under AddressSanitizer and UndefinedBehaviorSanitizer (no GPU): the CPU checker on
ragged shapes from exactly-sized heap buffers, and the CPU build of the device math over strided
sweeps of all bit patterns.  Each is a small C program built here with gcc and run on its own (a
sanitized library cannot be loaded into this interpreter)."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
FLAGS = ["-std=gnu11", "-O1", "-g", "-fopenmp", "-ffp-contract=off", "-fno-fast-math", "-mavx2", "-mfma",
         "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-fno-omit-frame-pointer"]


@pytest.mark.parametrize("name", ["sanitize_oracle", "sanitize_crmath"])
def test_under_sanitizers(name, tmp_path):
    exe = str(tmp_path / name)
    build = subprocess.run(["gcc"] + FLAGS + [os.path.join(HERE, name + ".c"), "-o", exe, "-lm"], capture_output=True, text=True)
    assert build.returncode == 0, build.stderr
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1", OMP_NUM_THREADS="4")
    env.pop("LD_PRELOAD", None)  # (the sanitizer runtime must come first in the program's own library list)
    run = subprocess.run([exe], capture_output=True, text=True, env=env, timeout=600)
    assert run.returncode == 0 and run.stdout.strip() == "ok", run.stdout + run.stderr
