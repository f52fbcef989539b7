"""The host side of the library under AddressSanitizer + UndefinedBehaviorSanitizer (host pass only, no GPU): layout
offset functions brute-forced for bijectivity (three formats, contiguous and paged), the format helpers swept, and the
validation halves of the entry points called with host-built descriptors.  tests/cpp/host_check.cpp is the program;
`make -C vesper_amd/csrc host_check` builds it (also done by __graft_entry__.build())."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_host_side_under_sanitizers():
    exe = os.path.join(ROOT, "tests", "cpp", "host_check")
    # always through make: incremental, so it costs nothing when the binary is newer than every source it is built from
    subprocess.check_call(["make", "-C", os.path.join(ROOT, "vesper_amd", "csrc"), "-j8", "host_check"],
                          stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="halt_on_error=1:print_stacktrace=1")
    r = subprocess.run([exe], capture_output=True, text=True, timeout=300, env=env)
    assert r.returncode == 0, (r.stdout[-3000:], r.stderr[-3000:])
    assert "host checks passed" in r.stdout
    assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr, r.stderr[-3000:]
