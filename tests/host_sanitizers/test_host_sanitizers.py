"""Host code of the library under AddressSanitizer + UndefinedBehaviorSanitizer and
under ThreadSanitizer.

Two small native drivers (beside this file) include a host-only translation unit
of the library each, run it on seeded random inputs against a plain model, and
are built here with clang's sanitizers (statically linked runtime).  GPU code is
not involved and nothing here is marked gpu: sanitizer builds belong on the CPU."""
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CLANG = shutil.which("clang++", path="/opt/rocm/llvm/bin") or shutil.which("clang++")
pytestmark = pytest.mark.skipif(CLANG is None, reason="no clang++ for a sanitizer build")


SANITIZERS = [pytest.param(("-fsanitize=address,undefined", "-fno-sanitize-recover=undefined"),
                           id="asan-ubsan"),
              pytest.param(("-fsanitize=thread",), id="tsan")]


def build_and_run(tmp_path, driver, sanitizer, extra=()):
    exe = str(tmp_path / "driver")
    cmd = [CLANG, "-std=c++17", "-O1", "-g", *sanitizer, "-fno-omit-frame-pointer",
           "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", "-I" + os.path.join(ROOT, "include"),
           "-I" + os.path.join(ROOT, "flexkv_amd", "csrc"), *extra,
           os.path.join(HERE, driver), "-o", exe, "-pthread", "-ldl"]
    subprocess.run(cmd, check=True, capture_output=True, text=True)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:verify_asan_link_order=0",
               TSAN_OPTIONS="halt_on_error=1", TMPDIR=str(tmp_path))
    r = subprocess.run([exe], capture_output=True, text=True, env=env, timeout=600)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-4000:]
    return r.stdout


@pytest.mark.parametrize("sanitizer", SANITIZERS)
def test_ssd_engine_under_sanitizers(tmp_path, sanitizer):
    out = build_and_run(tmp_path, "ssd_sanitizer_driver.cpp", sanitizer)
    assert "240 transfers round-tripped" in out


@pytest.mark.parametrize("sanitizer", SANITIZERS)
def test_host_row_copies_under_sanitizers(tmp_path, sanitizer):
    out = build_and_run(tmp_path, "host_copy_sanitizer_driver.cpp", sanitizer, extra=("-mavx2",))
    assert "400 scatter/gather pairs and 300 crew gathers" in out


@pytest.mark.parametrize("sanitizer", SANITIZERS)
def test_layerwise_poll_loop_under_sanitizers(tmp_path, sanitizer):
    """The polling loop of the layerwise restore (fkv_poll.h) on scripted event
    statuses: in-order announcements, a device error ends it without announcing what
    is left, a stop request ends it."""
    out = build_and_run(tmp_path, "poll_loop_driver.cpp", sanitizer)
    assert "ok: 301 scripted polls" in out


@pytest.mark.parametrize("sanitizer", SANITIZERS)
def test_batch_gate_of_a_gathered_restore_under_sanitizers(tmp_path, sanitizer):
    """The gate between the thread that launches a gathered layerwise restore batch by batch
    and its consumers (fkv_gate.h): scripted launchers that sometimes give up part-way,
    blocking waiters and the polling loop, 200 runs through one gate."""
    out = build_and_run(tmp_path, "batch_gate_driver.cpp", sanitizer)
    assert "ok: 200 scripted restores through the gate" in out


LIBRARY_HOST_SOURCES = ["fkv_core", "fkv_ce", "fkv_host", "fkv_host_copy", "fkv_tp_group",
                        "fkv_layerwise", "fkv_ipc", "fkv_ssd", "fkv_transform", "fkv_ranges",
                        "fkv_linkboard", "fkv_policy", "fkv_staged_restore"]


_LIBRARY_OBJECTS = {}   # sanitizer flags -> objects of the library over the emulated runtime


def _compile(cmd):
    subprocess.run(cmd, check=True, capture_output=True, text=True)


def build_over_emulated_runtime(tmp_path, driver, sanitizer, defines=()):
    """Every host translation unit of the library, the emulated HIP runtime (streams as
    threads, events as counters, the kernels as memcpy loops), the oracle's C file (the model
    of the thread-group cases) and a driver, compiled with the sanitizer and linked into one
    program.  The library's objects are built once per sanitizer and test session."""
    from concurrent.futures import ThreadPoolExecutor
    csrc = os.path.join(ROOT, "flexkv_amd", "csrc")
    flags = [CLANG, "-std=c++17", "-O1", "-g", *sanitizer, "-fno-omit-frame-pointer", "-mavx2",
             "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", "-I" + os.path.join(ROOT, "include"),
             "-I" + csrc]
    key = tuple(sanitizer)
    if key not in _LIBRARY_OBJECTS:
        import tempfile
        where = tempfile.mkdtemp(prefix="fkv_emulated_", dir=str(tmp_path.parent))
        units = [os.path.join(csrc, f + ".cpp") for f in LIBRARY_HOST_SOURCES]
        units.append(os.path.join(HERE, "emulated_hip_runtime.cpp"))
        objects = [os.path.join(where, os.path.basename(u)[:-4] + ".o") for u in units]
        jobs = [flags + ["-c", u, "-o", o] for u, o in zip(units, objects)]
        oracle = os.path.join(where, "fkv_oracle.o")
        jobs.append([shutil.which("clang", path=os.path.dirname(CLANG)) or "clang", "-O1", "-g",
                     *sanitizer, "-fno-omit-frame-pointer", "-c",
                     os.path.join(ROOT, "oracle", "fkv_oracle.c"), "-o", oracle])
        with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 2)) as pool:
            list(pool.map(_compile, jobs))
        _LIBRARY_OBJECTS[key] = objects + [oracle]
    source = driver if os.path.isabs(driver) else os.path.join(HERE, driver)
    obj = str(tmp_path / "driver.o")
    _compile(flags + [*defines, "-c", source, "-o", obj])
    exe = str(tmp_path / "driver")
    _compile([CLANG, *sanitizer, *_LIBRARY_OBJECTS[key], obj, "-o", exe, "-pthread", "-ldl"])
    return exe


@pytest.mark.parametrize("sanitizer", SANITIZERS)
def test_whole_host_side_over_an_emulated_runtime_under_sanitizers(tmp_path, sanitizer):
    """Layerwise restores with one, two and four ranks on every route and engine, pinned and
    pageable pools, both notify modes with eventfds, consumers gated per layer, restores that
    give up part-way; plain puts and gets on the kernel path and through every copy-engine
    strategy; the thread group of a tensor-parallel engine in every shared-KV mode and with
    head slices (against the oracle's rank plan); puts and gets from several threads at once;
    restores and transfers during which the runtime refuses allocations, streams, events,
    copies, launches or event records at seeded points (they fail or are made up for, and the
    next one is whole):
    the library's host code as it is shipped, over a HIP runtime made of threads, every byte
    against a plain model.  The library keeps per-stream events and staging memory until the
    process ends, so leak checking is off for this program."""
    exe = build_over_emulated_runtime(tmp_path, "layerwise_emulated_driver.cpp", sanitizer)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:verify_asan_link_order=0",
               TSAN_OPTIONS="halt_on_error=1", TMPDIR=str(tmp_path))
    r = subprocess.run([exe, "80", "40"], capture_output=True, text=True, env=env, timeout=900)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-6000:]
    assert ("ok: 80 groups of layerwise restores, 40 sets of transfers, 40 thread groups and "
            "40 bursts of concurrent calls") in r.stdout
    assert "runtime calls refused on request" in r.stdout


@pytest.mark.parametrize("sanitizer", SANITIZERS)
def test_native_consumers_over_an_emulated_runtime_under_sanitizers(tmp_path, sanitizer):
    """The two native consumers of the C ABI (tests/native), which the GPU suite runs against
    the shipped library, here linked with the library's host code over the emulated runtime:
    every entry point that does not live beside the kernels (kernel path, each copy-engine
    strategy, several transfers in one call, thread group, layerwise restore on each route
    with eventfds, two-group restore with a sidecar, layout transform, the board processes
    share), and a put thread next to a get thread."""
    native = os.path.join(ROOT, "tests", "native")
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:verify_asan_link_order=0",
               TSAN_OPTIONS="halt_on_error=1", TMPDIR=str(tmp_path))
    for source, args, expect in (("abi_roundtrip_driver.cpp", [], "ok: 33 cases through the C ABI"),
                                 ("two_way_driver.cpp", ["0.3", "8"], "ok: puts alone")):
        sub = tmp_path / source[:-4]
        sub.mkdir()
        exe = build_over_emulated_runtime(sub, os.path.join(native, source), sanitizer,
                                          defines=("-DFKV_EMULATED_RUNTIME",))
        r = subprocess.run([exe, *args], capture_output=True, text=True, env=env, timeout=900)
        assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-6000:]
        assert expect in r.stdout, r.stdout[-2000:]
