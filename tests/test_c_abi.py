"""The header is a plain C header and the library a plain C ABI: a C11 program (gcc -pedantic -Werror)
includes include/fv_sdpa_hip.h, links libfv_sdpa_hip.so and calls host-only entry points. No GPU."""
import os
import shutil
import subprocess

import pytest

from util import ROOT


def _host_calls(tmp_path, pkg):
    exe = str(tmp_path / "host_calls")
    subprocess.check_call(["gcc", "-std=c11", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(ROOT, "include"),
                           os.path.join(ROOT, "tests", "c_abi", "host_calls.c"), "-o", exe, "-L", pkg, "-lfv_sdpa_hip",
                           "-Wl,-rpath," + pkg, "-Wl,-rpath,/opt/rocm/lib"])
    out = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, (out.returncode, out.stdout, out.stderr)
    line = out.stdout.strip()
    assert "supported=10 " in line and "tiles=624 topk=125 " in line
    assert "kvmove=30,30,60,0 " in line              # wan/causal.rs:901-906
    assert "block_causal=1170,2,0 " in line          # rt/attn.rs:630-645: 3 frames of 390 tokens, window 6 frames = 2 blocks
    assert "shards=0,6,6,5 " in line                 # rt/sp.rs:66-74
    assert "backend=1 route=2:1,2 " in line
    assert "local_attn_size=-1 keeps a 21-frame KV window" in line   # the refused plan's message


@pytest.mark.skipif(shutil.which("gcc") is None, reason="no C compiler")
def test_header_compiles_as_c_and_links(tmp_path):
    _host_calls(tmp_path, os.path.join(ROOT, "fastvideo-rs_amd"))


@pytest.mark.skipif(shutil.which("gcc") is None or shutil.which("hipcc") is None, reason="no compilers")
def test_host_layer_is_clean_under_the_undefined_behaviour_sanitizer(tmp_path):
    """`make ubsan` builds the library with its host code under -fsanitize=undefined in trap mode (device code
    as always) into a temp dir; the C program above and every host-only test of the C ABI (geometry, KV-cache
    plans, tile walks, routes, argument refusals, known answers) then run against that build in child
    processes: undefined behaviour anywhere in the host layer kills the child with SIGILL."""
    import sys

    out = tmp_path / "ubsan"
    csrc = os.path.join(ROOT, "fastvideo-rs_amd", "csrc")
    b = subprocess.run(["make", "-C", csrc, "-j8", "ubsan", f"UBSAN_DIR={out}"], capture_output=True, text=True)
    assert b.returncode == 0, b.stderr[-3000:]
    so = out / "libfv_sdpa_hip.so"
    assert so.exists()
    dump = subprocess.run(["objdump", "-d", str(so)], capture_output=True, text=True).stdout
    assert dump.count("ud1") + dump.count("ud2") > 100      # the traps are in: the flags reached the host pass
    _host_calls(tmp_path, str(out))
    env = dict(os.environ, FV_SDPA_HIP_LIB=str(so))
    r = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-m", "not gpu", "-p", "no:cacheprovider",
                        os.path.join(ROOT, "tests", "test_host_abi.py"),
                        os.path.join(ROOT, "tests", "test_golden_known_answers.py"),
                        os.path.join(ROOT, "tests", "test_oracle_kv_cache.py")],
                       capture_output=True, text=True, env=env, cwd=ROOT, timeout=900)
    assert r.returncode == 0, (r.returncode, r.stdout[-3000:], r.stderr[-2000:])
    assert " passed" in r.stdout


def test_oracle_c_functions_are_clean_under_address_and_undefined_sanitizers(tmp_path):
    """The checker itself is checked: every C function of the oracle runs on odd small shapes in a
    native build with -fsanitize=address,undefined (leak check on); any report aborts the driver."""
    exe = str(tmp_path / "oracle_sanitize")
    build = subprocess.run(["gcc", "-O1", "-g", "-std=c11", "-fopenmp", "-ffp-contract=off", "-fsanitize=address,undefined",
                            "-fno-sanitize-recover=all", "-I", os.path.join(ROOT, "oracle"),
                            os.path.join(ROOT, "tests", "c_abi", "oracle_sanitize.c"), os.path.join(ROOT, "oracle", "fv_oracle.c"),
                            "-o", exe, "-lm"], capture_output=True, text=True)
    if build.returncode != 0 and ("asan" in build.stderr.lower() or "sanitize" in build.stderr.lower()):
        pytest.skip("this gcc has no sanitizer runtimes")
    assert build.returncode == 0, build.stderr[-2000:]
    env = dict(os.environ)
    env["ASAN_OPTIONS"] = "detect_leaks=1:verify_asan_link_order=0"
    out = subprocess.run([exe], capture_output=True, text=True, timeout=120, env=env)
    assert out.returncode == 0 and "oracle sanitizer run: ok" in out.stdout, (out.returncode, out.stdout[-500:], out.stderr[-3000:])
