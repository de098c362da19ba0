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


LIBRARY_KERNEL_SOURCES = ["fkv_kernels", "fkv_noalloc", "fkv_staging"]

_LIBRARY_OBJECTS = {}   # sanitizer flags -> objects of the library's host code
_DEVICE_OBJECTS = {}    # (sanitizer flags, kernels from source) -> emulated runtime and kernels


def _compile(cmd):
    subprocess.run(cmd, check=True, capture_output=True, text=True)


def kernel_source_as_cpp(name, where):
    """A kernel source of the library as a C++ file for the CPU device model
    (cpu_device_model.h, included first): the three places where the device language has no
    C++ spelling are rewritten, each checked to be there as often as expected, so that a
    change of the source that this would miss fails here instead."""
    text = open(os.path.join(ROOT, "flexkv_amd", "csrc", name + ".hip")).read()

    def rewrite(old, new, count):
        nonlocal text
        assert text.count(old) == count, (name, old, text.count(old))
        text = text.replace(old, new)

    if name == "fkv_kernels":
        # dynamically sized LDS: one array per workgroup, handed out by the model
        rewrite("extern __shared__ uint64_t lds[];",
                "uint64_t *lds = static_cast<uint64_t *>(cpu_device_model::dynamic_lds());", 2)
        rewrite('asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(v));',
                "v = cpu_device_model::xcc_id();", 1)
        # the three entry points that time the device keep their stand-ins
        rewrite("int fkv_streams_run_concurrently(", "int fkv_streams_run_concurrently_timed(", 1)
        rewrite("int fkv_measure_hbm_rate(", "int fkv_measure_hbm_rate_timed(", 1)
        rewrite("int fkv_streams_hand_over_us(", "int fkv_streams_hand_over_us_timed(", 1)
    path = os.path.join(where, name + ".cpp")
    with open(path, "w") as f:
        f.write(text)
    return path


def build_over_emulated_runtime(tmp_path, driver, sanitizer, defines=(), kernels_from_source=False):
    """Every host translation unit of the library, the emulated HIP runtime (streams as
    threads, events as counters), the oracle's C file (the model of the thread-group cases)
    and a driver, compiled with the sanitizer and linked into one program.  The kernels are
    memcpy loops of the emulated runtime, or (`kernels_from_source`) the library's own kernel
    sources compiled for the CPU device model: every work-item a host thread, so that the
    sanitizer sees the addresses the kernels compute.  Objects are built once per sanitizer
    and test session."""
    from concurrent.futures import ThreadPoolExecutor
    import tempfile
    csrc = os.path.join(ROOT, "flexkv_amd", "csrc")
    flags = [CLANG, "-std=c++17", "-O1", "-g", *sanitizer, "-fno-omit-frame-pointer", "-mavx2",
             "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", "-I" + os.path.join(ROOT, "include"),
             "-I" + csrc, "-I" + HERE]
    key = tuple(sanitizer)
    jobs = []
    if key not in _LIBRARY_OBJECTS:
        where = tempfile.mkdtemp(prefix="fkv_emulated_", dir=str(tmp_path.parent))
        units = [os.path.join(csrc, f + ".cpp") for f in LIBRARY_HOST_SOURCES]
        objects = [os.path.join(where, os.path.basename(u)[:-4] + ".o") for u in units]
        jobs += [flags + ["-c", u, "-o", o] for u, o in zip(units, objects)]
        oracle = os.path.join(where, "fkv_oracle.o")
        jobs.append([shutil.which("clang", path=os.path.dirname(CLANG)) or "clang", "-O1", "-g",
                     *sanitizer, "-fno-omit-frame-pointer", "-c",
                     os.path.join(ROOT, "oracle", "fkv_oracle.c"), "-o", oracle])
        _LIBRARY_OBJECTS[key] = objects + [oracle]
    if (key, kernels_from_source) not in _DEVICE_OBJECTS:
        where = tempfile.mkdtemp(prefix="fkv_device_", dir=str(tmp_path.parent))
        mode = ["-DFKV_KERNELS_FROM_SOURCE"] if kernels_from_source else []
        objects = [os.path.join(where, "emulated_hip_runtime.o")]
        jobs.append(flags + mode + ["-c", os.path.join(HERE, "emulated_hip_runtime.cpp"),
                                    "-o", objects[0]])
        if kernels_from_source:
            for name in LIBRARY_KERNEL_SOURCES:
                objects.append(os.path.join(where, name + ".o"))
                jobs.append(flags + mode + ["-include", os.path.join(HERE, "cpu_device_model.h"),
                                            "-c", kernel_source_as_cpp(name, where),
                                            "-o", objects[-1]])
        _DEVICE_OBJECTS[(key, kernels_from_source)] = objects
    if jobs:
        with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 2)) as pool:
            list(pool.map(_compile, jobs))
    source = driver if os.path.isabs(driver) else os.path.join(HERE, driver)
    obj = str(tmp_path / "driver.o")
    _compile(flags + [*defines, "-c", source, "-o", obj])
    exe = str(tmp_path / "driver")
    _compile([CLANG, *sanitizer, *_LIBRARY_OBJECTS[key],
              *_DEVICE_OBJECTS[(key, kernels_from_source)], obj, "-o", exe, "-pthread", "-ldl"])
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
    for source, args, expect in (("abi_roundtrip_driver.cpp", [], "ok: 34 cases through the C ABI"),
                                 ("two_way_driver.cpp", ["0.3", "8"], "ok: puts alone")):
        sub = tmp_path / source[:-4]
        sub.mkdir()
        exe = build_over_emulated_runtime(sub, os.path.join(native, source), sanitizer,
                                          defines=("-DFKV_EMULATED_RUNTIME",))
        r = subprocess.run([exe, *args], capture_output=True, text=True, env=env, timeout=900)
        assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-6000:]
        assert expect in r.stdout, r.stdout[-2000:]


@pytest.mark.parametrize("sanitizer", SANITIZERS)
def test_kernel_sources_on_a_cpu_device_model_under_sanitizers(tmp_path, sanitizer):
    """The same two programs with the library's kernels compiled from their own sources for a
    CPU model of the device (cpu_device_model.h: a workgroup is a crew of host threads,
    __syncthreads a barrier, the atomics host atomics, XCD ids dealt in turn with a start that
    moves from launch to launch): AddressSanitizer checks every address the gather/scatter
    kernel computes on every route (whole slices, short last slices, packed chunks, several
    jobs in one launch, fixed shares, claimed ranges, launches confined to some XCDs and their
    safety net), ThreadSanitizer the order among work-items; the launch shaping, the plan
    upload, the entry point that allocates nothing and the compressed-staging kernels run as
    shipped (36 cases of the ABI driver instead of 34)."""
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:verify_asan_link_order=0",
               TSAN_OPTIONS="halt_on_error=1", TMPDIR=str(tmp_path))
    sub = tmp_path / "restores"
    sub.mkdir()
    exe = build_over_emulated_runtime(sub, "layerwise_emulated_driver.cpp", sanitizer,
                                      kernels_from_source=True)
    r = subprocess.run([exe, "6", "4"], capture_output=True, text=True, env=env, timeout=900)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-6000:]
    assert "ok: 6 groups of layerwise restores, 4 sets of transfers" in r.stdout
    assert "kernels from their sources:" in r.stdout
    sub = tmp_path / "abi"
    sub.mkdir()
    exe = build_over_emulated_runtime(
        sub, os.path.join(ROOT, "tests", "native", "abi_roundtrip_driver.cpp"), sanitizer,
        defines=("-DFKV_EMULATED_RUNTIME", "-DFKV_KERNELS_FROM_SOURCE"), kernels_from_source=True)
    r = subprocess.run([exe], capture_output=True, text=True, env=env, timeout=900)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-6000:]
    assert "ok: 36 cases through the C ABI" in r.stdout, r.stdout[-2000:]


@pytest.mark.parametrize("sanitizer,launches", [(SANITIZERS[0].values[0], 40),
                                                (SANITIZERS[1].values[0], 20)],
                         ids=["asan-ubsan", "tsan"])
def test_gather_scatter_kernel_shapes_on_a_cpu_device_model(tmp_path, sanitizer, launches):
    """The gather/scatter kernel by itself, launched through the library's own shaping code
    with seeded arguments over the space of shapes (vector widths 1-16, whole slices, a short
    last slice, packed chunks, the deep unroll, up to 1024 (layer, kv) pairs, more positions
    than an id tile, with and without id lists, both store kinds, fixed shares, claimed ranges,
    confined launches with dirty counters, one to four jobs a launch).  Tables, id lists and
    chunk regions are allocations of exactly the size the kernel may touch, so one vector too
    far is a sanitizer report; every destination byte is compared with a plain model.
    400 launches of the same program were run once by hand (clean); the suite runs fewer."""
    exe = build_over_emulated_runtime(tmp_path, "copy_kernel_model_driver.cpp", sanitizer,
                                      kernels_from_source=True)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:verify_asan_link_order=0",
               TSAN_OPTIONS="halt_on_error=1", TMPDIR=str(tmp_path))
    r = subprocess.run([exe, str(launches)], capture_output=True, text=True, env=env, timeout=900)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-6000:]
    assert "ok: %d launches of the gather/scatter kernel on the CPU device model" % launches in r.stdout
