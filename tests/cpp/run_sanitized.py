#!/usr/bin/env python3
"""Builds the host library and the C++ test programs with a sanitizer and runs the CPU suites.

    python tests/cpp/run_sanitized.py thread|address|undefined [build_dir] [--build-only | --run-only] [--gpu | --stand-in] [--repeat=N]

Host code only (g++ -fsanitize=...); libtphip.so is used as built. With --gpu the suites of the
device channels run instead of the CPU ones (on a machine with a GPU; --build-only on one machine
and --run-only on another share a build directory; next to the HIP runtime AddressSanitizer needs
ASAN_OPTIONS=use_sigaltstack=0:protect_shadow_gap=0:detect_leaks=0, and ThreadSanitizer does not
work at all: the runtime finds no device under its address-space layout). With --stand-in the same
device-channel suites run on the CPU against tests/cpp/fake_tphip.cc, the host-only stand-in for
libtphip.so built with the same sanitizer (streams are threads, copies are memcpy, events and signal
words are real synchronisation): the channels' host logic, which ThreadSanitizer cannot see next to
the HIP runtime, is checked there, a missing wait between a copy and its consumer included; the
executor cases (unit_tests loops) run in every mode. Not collected by pytest: a
full pass takes several minutes. The shm transport tells ThreadSanitizer about the hand-off
through its rings (two mappings of one segment inside a process), so a clean run reports
nothing; any "WARNING: ThreadSanitizer" / "ERROR: AddressSanitizer" line fails the run.
With --repeat=N every suite runs up to N times and stops at its first bad turn; a turn that is
still running after three minutes is asked for the call stacks of all its threads and ended (a
hang that shows once in a hundred runs is found this way: the sanitizers' slower, differently
skewed timing brings out orders of events that a plain build almost never takes).
"""
import os
import signal
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from tensorpipe_amd import build as tp_build  # noqa: E402

# (program, suite, stock wire format)
SUITES = [("channel_tests", "xth", False), ("channel_tests", "basic", False),
          ("pipe_tests", "cpu_same_process", False), ("pipe_tests", "cpu_two_process", False),
          ("pipe_tests", "cpu_same_process", True), ("pipe_tests", "cpu_two_process", True)]


GPU_SUITES = [("channel_tests", "hip_xth", False), ("channel_tests", "hip_ipc", False),
              ("channel_tests", "hip_ipc_outbox", False), ("channel_tests", "hip_basic", False),
              ("pipe_tests", "same_process", False), ("pipe_tests", "two_process", False),
              ("pipe_tests", "two_process", True)]


STAND_IN_SUITES = GPU_SUITES + [("channel_tests", "hip_ipc_gated", False), ("channel_tests", "hip_ipc_messages", False),
                                ("channel_tests", "hip_basic_host_ring", False),
                                ("channel_tests", "hip_basic_small_ring", False)]


REPEAT = 1


def main():
    global REPEAT
    words = [a for a in sys.argv[1:] if not a.startswith("--")]
    options = {a for a in sys.argv[1:] if a.startswith("--")}
    for a in options:
        if a.startswith("--repeat="):
            REPEAT = max(1, int(a.split("=", 1)[1]))
    san = words[0] if words else "thread"
    out = os.path.abspath(words[1]) if len(words) > 1 else tempfile.mkdtemp(prefix=f"tp_{san}_")
    os.makedirs(out, exist_ok=True)
    if "--run-only" not in options:
        build(san, out)
    if "--build-only" in options:
        return
    if "--gpu" in options:
        sys.exit(1 if run_suites(out, GPU_SUITES) else 0)
    if "--stand-in" in options:
        env = dict(os.environ, LD_LIBRARY_PATH=os.path.join(out, "fake"))
        bad = run_suites(out, STAND_IN_SUITES, env)
        bad += run_unit(out, ["loops"], env)
        bad += run_conformance(out, env)
        sys.exit(1 if bad else 0)
    run_cpu(out)


def build(san, out):
    flags = ["-O1", "-g", "-std=c++17", "-fPIC", f"-fsanitize={san}", "-fno-omit-frame-pointer", "-pthread",
             f"-I{tp_build.INCLUDE}", f"-I{tp_build.CSRC}"]
    objs = [os.path.join(out, s.replace("/", "_") + ".o") for s in tp_build.HOST_SOURCES]

    def compile_one(pair):
        src, obj = pair
        subprocess.run(["g++", *flags, "-c", os.path.join(tp_build.CSRC, src), "-o", obj], check=True)

    with ThreadPoolExecutor(max_workers=8) as pool:
        list(pool.map(compile_one, zip(tp_build.HOST_SOURCES, objs)))
    # the stand-in for libtphip.so, sanitized like the rest (chosen at run time by LD_LIBRARY_PATH)
    os.makedirs(os.path.join(out, "fake"), exist_ok=True)
    subprocess.run(["g++", *flags, "-shared", os.path.join(ROOT, "tests", "cpp", "fake_tphip.cc"), "-o",
                    os.path.join(out, "fake", "libtphip.so")], check=True)
    lib = os.path.join(out, "libtensorpipe_amd.so")
    subprocess.run(["g++", "-shared", f"-fsanitize={san}", "-pthread", "-o", lib, *objs, f"-L{tp_build.LIB}",
                    "-ltphip", f"-Wl,-rpath,{tp_build.LIB}"], check=True)
    for prog in sorted({p for p, _, _ in SUITES} | {"unit_tests"}):
        subprocess.run(["g++", *flags, os.path.join(ROOT, "tests", "cpp", prog + ".cc"), "-o",
                        os.path.join(out, prog), f"-L{out}", "-ltensorpipe_amd", f"-L{tp_build.LIB}", "-ltphip",
                        f"-Wl,-rpath,{out}", f"-Wl,-rpath,{tp_build.LIB}"], check=True)
    build_conformance(san, out, flags)


# The conformance program: the channels inside the unmodified TensorPipe of libtorch_cpu.so, where
# every thread but the event poller's is a stranger to this library. AddressSanitizer only: the
# stock library is not instrumented, and ThreadSanitizer then reports its internals.
CONFORMANCE_MODES = [["same_process"], ["two_process", "hip_ipc"], ["two_process", "hip_basic"],
                     ["to_self", "hip_xth", "300"], ["to_self", "hip_basic", "300"],
                     ["native_peer", "hip_xth"], ["native_peer", "hip_ipc"], ["native_peer", "hip_basic"],
                     ["native_peer", "hip_basic", "shm"], ["unmodified_peer"]]


def build_conformance(san, out, flags):
    found = tp_build.stock_tensorpipe()
    if san != "address" or found is None:
        return
    inc, lib = found
    stock_first = [f for f in flags if not f.startswith("-I")]
    subprocess.run(["g++", *stock_first, f"-I{inc}", f"-I{tp_build.INCLUDE}", f"-I{tp_build.CSRC}",
                    os.path.join(tp_build.CSRC, "bridge", "stock_adapter.cc"),
                    os.path.join(ROOT, "tests", "cpp", "stock_conformance.cc"),
                    "-o", os.path.join(out, "stock_conformance"), f"-L{out}", "-ltensorpipe_amd",
                    f"-L{tp_build.LIB}", "-ltphip", f"-L{lib}", "-ltorch_cpu", "-lc10",
                    f"-Wl,-rpath,{out}", f"-Wl,-rpath,{tp_build.LIB}", f"-Wl,-rpath,{lib}"], check=True)


def run_conformance(out, env):
    prog = os.path.join(out, "stock_conformance")
    if not os.path.exists(prog):
        return 0
    bad = 0
    env = dict(env, ASAN_OPTIONS=(env.get("ASAN_OPTIONS", "") + ":detect_leaks=0").lstrip(":"))
    for args in CONFORMANCE_MODES:
        text, stuck = run_once([prog, *args], env, 600)
        results = [l for l in text.splitlines() if l.startswith("RESULT")]
        failed = [l for l in results if " OK" not in l]
        reports = sanitizer_lines(text)
        print(f"stock_conformance {' '.join(args)}: {len(results)} results, {len(failed)} failed, "
              f"{len(reports)} sanitizer reports{', STUCK: stacks below' if stuck else ''}")
        for l in failed + reports[:5]:
            print("   ", l[:200])
        if stuck:
            print(text[-6000:])
        bad += len(failed) + len(reports) + (0 if results else 1) + (1 if stuck else 0)
        sys.stdout.flush()
    return bad


def run_unit(out, args, env=None):
    proc = subprocess.run([os.path.join(out, "unit_tests"), *args],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=900, env=env)
    reports = sanitizer_lines(proc.stdout)
    lines = proc.stdout.strip().splitlines()
    ok = proc.returncode == 0 and bool(lines) and lines[-1].startswith("OK")
    print(f"unit_tests {args[0]}: {'ok' if ok else 'FAILED'}, {len(reports)} sanitizer reports")
    for l in reports[:5] + ([] if ok else lines[-5:]):
        print("   ", l[:200])
    sys.stdout.flush()
    return (0 if ok else 1) + len(reports)


def sanitizer_lines(text):
    """The lines with which a sanitizer announces a finding (thread, address, leak, undefined behaviour)."""
    marks = ("WARNING: ThreadSanitizer", "ERROR: AddressSanitizer", "ERROR: LeakSanitizer", "runtime error:")
    return [l for l in text.splitlines() if any(m in l for m in marks)]


def run_once(cmd, env, limit):
    """Output of `cmd`, and whether it had to be ended. A program that is still running after
    `limit` seconds is asked for its threads' stacks (SIGUSR1, tests/cpp/support.h) and killed."""
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    try:
        text, _ = proc.communicate(timeout=limit)
        return text, False
    except subprocess.TimeoutExpired:
        proc.send_signal(signal.SIGUSR1)
        time.sleep(5)
        proc.kill()
        text, _ = proc.communicate()
        return text, True


def run_suites(out, suites, base_env=None):
    bad = 0
    for prog, suite, stock_wire in suites:
        env = dict(base_env or os.environ, TP_STOCK_WIRE="1") if stock_wire else base_env
        label = f"{prog} --suite {suite}{' (stock wire format)' if stock_wire else ''}"
        for turn in range(REPEAT):
            text, stuck = run_once([os.path.join(out, prog), "--suite", suite], env, 1800 if REPEAT == 1 else 180)
            results = [l for l in text.splitlines() if l.startswith("RESULT")]
            failed = [l for l in results if " OK" not in l]
            reports = sanitizer_lines(text)
            if stuck or failed or reports or not results:
                break
        where = f" (turn {turn + 1} of {REPEAT})" if REPEAT > 1 else ""
        print(f"{label}{where}: {len(results)} results, {len(failed)} failed, {len(reports)} sanitizer reports"
              f"{', STUCK: stacks below' if stuck else ''}")
        for l in failed + reports[:5]:
            print("   ", l[:200])
        if stuck:
            print(text[-6000:])
        bad += len(failed) + len(reports) + (0 if results else 1) + (1 if stuck else 0)
        sys.stdout.flush()
    return bad


def run_cpu(out):
    bad = run_suites(out, SUITES)
    bad += run_unit(out, ["loops"])
    # random bytes where a pipe's first packets belong
    for seed in (11, 12, 13):
        proc = subprocess.run([os.path.join(out, "unit_tests"), "garbage", str(seed), "150"],
                              stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
        reports = sanitizer_lines(proc.stdout)
        ok = proc.returncode == 0 and proc.stdout.strip().endswith("OK")
        print(f"unit_tests garbage {seed}: {'ok' if ok else 'FAILED'}, {len(reports)} sanitizer reports")
        for l in reports[:5]:
            print("   ", l[:200])
        bad += (0 if ok else 1) + len(reports)
    # a peer that wrote and left before the reads were posted
    proc = subprocess.run([os.path.join(out, "unit_tests"), "departed_peer"],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    reports = sanitizer_lines(proc.stdout)
    ok = proc.returncode == 0 and proc.stdout.strip().endswith("OK")
    print(f"unit_tests departed_peer: {'ok' if ok else 'FAILED'}, {len(reports)} sanitizer reports")
    for l in reports[:5]:
        print("   ", l[:200])
    bad += (0 if ok else 1) + len(reports)
    # the stock-protocol decoder on whole, cut and bent frames, and two of its endpoints talking
    vectors = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "golden", "stock_wire_vectors.txt")
    for args in (["nop_wire", vectors], ["compat_pipe"], ["tcp"], ["shm_stock"], ["shm_stock_hostile_peer"],
                 ["transport_suite", "shm"], ["transport_suite", "shm_stock"], ["transport_suite", "tcp"]):
        proc = subprocess.run([os.path.join(out, "unit_tests"), *args],
                              stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
        reports = sanitizer_lines(proc.stdout)
        ok = proc.returncode == 0 and proc.stdout.strip().splitlines()[-1].startswith("OK")
        print(f"unit_tests {' '.join(a for a in args if not os.path.isabs(a))}: {'ok' if ok else 'FAILED'}, {len(reports)} sanitizer reports")
        for l in reports[:5] + ([] if ok else proc.stdout.strip().splitlines()[-8:]):
            print("   ", l[:200])
        bad += (0 if ok else 1) + len(reports)
    sys.exit(1 if bad else 0)


if __name__ == "__main__":
    main()
