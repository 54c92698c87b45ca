"""tch_TorchColShutdown while other threads are inside the shared-memory communicator (CPU only).

tests/host/shutdown_race.cc is built against the host runtime's own sources (host code only, no device pass)
once with ThreadSanitizer and once with AddressSanitizer, and run: a control thread and two receivers blocked in
tch_mq_timed_get, a sender in tch_mq_put / tch_train_info_set_field, and the main thread shutting the runtime
down under them, twenty times.  A use-after-unmap of the segment is a sanitizer report and a non-zero exit."""
import glob
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "sirius_amd", "csrc")


@pytest.mark.parametrize("sanitizer", ["thread", "address"])
def test_shutdown_under_blocked_waiters(tmp_path, sanitizer):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc")
    srcs = sorted(glob.glob(os.path.join(CSRC, "host", "*.cc"))) + [os.path.join(CSRC, "context.cc"),
                                                                    os.path.join(ROOT, "tests", "host", "shutdown_race.cc")]
    flags = ["-std=c++17", "-O1", "-g", "-x", "hip", "--offload-arch=gfx950", "--offload-host-only",
             "-Xarch_host", f"-fsanitize={sanitizer}", "-fno-omit-frame-pointer", "-I", os.path.join(ROOT, "include")]
    objs = []
    procs = []
    for s in srcs:
        o = str(tmp_path / (os.path.basename(s) + ".o"))
        objs.append(o)
        procs.append(subprocess.Popen([hipcc] + flags + ["-c", s, "-o", o], stdout=subprocess.PIPE, stderr=subprocess.STDOUT))
    for p in procs:
        out, _ = p.communicate()
        assert p.returncode == 0, out.decode()[-3000:]
    exe = str(tmp_path / "shutdown_race")
    link = subprocess.run([hipcc, f"-fsanitize={sanitizer}", "-fno-gpu-sanitize"] + objs + ["-o", exe, "-lpthread", "-lrt", "-lhsa-runtime64"],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    assert link.returncode == 0, link.stdout.decode()[-3000:]
    # the environment is passed on as it is; verify_asan_link_order=0 lets the sanitizer runtime start behind
    # whatever else the loader was asked to load first
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=1 exitcode=66",
               ASAN_OPTIONS="detect_leaks=0 exitcode=67 verify_asan_link_order=0")
    run = subprocess.run([exe, "20"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=240, env=env)
    text = run.stdout.decode()
    assert run.returncode == 0, text[-4000:]
    assert "rounds clean" in text
