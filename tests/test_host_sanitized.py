"""The host library's C (tensors, layers, model container, quantized weights, model / tensor /
quantized-weight files) compiled with AddressSanitizer, LeakSanitizer and UndefinedBehaviorSanitizer and
driven on the CPU device: object lifetimes and refused arguments, then the reference-written fixtures with
their truncations, bit flips and crafted headers (tests/host_sanitize_driver.c).  No GPU; a finding aborts."""
import glob
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)


def test_file_code_is_clean_under_asan_and_ubsan(tmp_path):
    exe = tmp_path / "host_sanitize_driver"
    srcs = sorted(glob.glob(os.path.join(ROOT, "axiom_amd", "csrc", "host", "*.c")))
    lib = os.path.join(ROOT, "axiom_amd", "lib")
    assert os.path.exists(os.path.join(lib, "libaxhip.so")), "build the libraries first (__graft_entry__.build())"
    cmd = ["gcc", "-std=gnu11", "-O1", "-g", "-fno-omit-frame-pointer", "-fsanitize=address,undefined",
           "-fno-sanitize-recover=undefined", "-I" + os.path.join(ROOT, "include"),
           os.path.join(HERE, "host_sanitize_driver.c")] + srcs + \
          ["-L" + lib, "-laxhip", "-Wl,-rpath," + lib, "-lm", "-lpthread", "-o", str(exe)]
    subprocess.run(cmd, check=True, capture_output=True, text=True)
    # ref_flatten.axm holds a layer type this library refuses: not a round-trip case
    files = [f for f in sorted(glob.glob(os.path.join(HERE, "golden", "ref_*.axm"))) if "flatten" not in f] + \
            [os.path.join(HERE, "golden", "ref_tensor.axt")]
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:detect_leaks=1:abort_on_error=0",
               UBSAN_OPTIONS="print_stacktrace=1")
    r = subprocess.run([str(exe), str(tmp_path / "scratch.bin")] + files, env=env, capture_output=True, text=True,
                       timeout=600)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-6000:]
    assert r.stdout.count("round trip ok") == len(files) and "api section: 0 findings" in r.stdout
