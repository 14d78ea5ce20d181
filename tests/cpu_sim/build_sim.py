"""Builds libophip_cpusim.so: the library's own host objects (operators-rs_amd/csrc/build/*.o, exactly those that go
into libophip.so) linked with its kernel sources compiled for the host (hip/hip_runtime.h, cpusim_core.h) and with a
stand-in for the HIP runtime (sim_runtime.cpp), so that the CPU tests can drive the whole library through its C ABI
without a GPU.  Test infrastructure only: nothing in the product builds, loads or knows this library.

For each code object of the library's Makefile (KERNELS) one translation unit is generated that includes the kernel
source inside a namespace of the module and registers every `extern "C" __global__` function it defines (found by
preprocessing the source with __global__ defined to a marker).  Objects are rebuilt when the text they are made from changes.

    python tests/cpu_sim/build_sim.py [out_dir [sanitizers]]      (default tests/cpu_sim/_build, none)

With sanitizers (e.g. `undefined`: UndefinedBehaviorSanitizer needs no preloading, so python can load the result) the
host sources are compiled here as well, with the same checks, instead of taking the Makefile's objects.
"""
import concurrent.futures
import hashlib
import os
import re
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(ROOT, "operators-rs_amd", "csrc")
KERNELS = os.path.join(CSRC, "kernels")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HOST_OBJECTS = ["handle", "ops", "random_sample", "mat_mul", "attention", "ops_more", "conv", "static_scratch"]
DEVICE_FLAGS = ["-std=c++20", "-O1", "-fPIC", "-x", "c++", "-I", HERE, "-I", KERNELS, "-DOPHIP_CPU_SIM=1", "-Wno-unused-value",
                "-Wno-pass-failed", "-Wno-unknown-attributes"]


def compiler():
    cxx = os.path.join(ROCM, "lib", "llvm", "bin", "clang++")
    if os.path.exists(cxx):
        return cxx
    return shutil.which("clang++")


def modules():
    """(module name, source file, extra defines) for every code object the library embeds (csrc/Makefile: KERNELS)."""
    text = open(os.path.join(CSRC, "Makefile")).read().replace("\\\n", " ")
    names = re.search(r"^KERNELS\s*:=\s*(.*)$", text, re.M).group(1).split()
    out = []
    for n in names:
        if n.endswith("_bf16"):
            out.append((n, os.path.join(KERNELS, n[:-5] + ".hip"), ["-DGEMM_ELEM_BF16"]))
        else:
            out.append((n, os.path.join(KERNELS, n + ".hip"), []))
    return out


def run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("%s\n%s" % (" ".join(cmd), (r.stdout + r.stderr)[-6000:]))
    return r.stdout


def digest(*parts):
    h = hashlib.sha256()
    for p in parts:
        h.update(p.encode() if isinstance(p, str) else p)
        h.update(b"\0")
    return h.hexdigest()


def compile_if_stale(cxx, flags, src, obj, preprocessed_text):
    """Compiles src -> obj unless obj was made from the same preprocessed text with the same flags."""
    stamp = obj + ".sha"
    want = digest(" ".join(flags), preprocessed_text)
    if os.path.exists(obj) and os.path.exists(stamp) and open(stamp).read() == want:
        return False
    run([cxx] + flags + ["-c", "-o", obj, src])
    open(stamp, "w").write(want)
    return True


def sanitizer_flags(sanitize):
    return ["-g", "-fsanitize=" + sanitize, "-fno-sanitize-recover=all", "-shared-libsan"] if sanitize else []


def build_module(cxx, out_dir, name, source, defines, sanitize=None):
    flags = DEVICE_FLAGS + defines + sanitizer_flags(sanitize)
    marked = run([cxx] + flags + ["-D__global__=CPUSIM_GLOBAL_MARK", "-E", "-P", source])
    kernels = re.findall(r"CPUSIM_GLOBAL_MARK\s+void\s+(\w+)\s*\(", marked)
    if not kernels:
        raise RuntimeError("no kernels found in " + source)
    tu = os.path.join(out_dir, "mod_%s.cpp" % name)
    # the launch's dynamic LDS, which the source only declares
    dynamic = re.findall(r"extern\s+thread_local\s+(\w+)\s+(\w+)\s*\[\s*\]\s*;", marked)
    # Everything of the module goes into a namespace of its own: on the GPU every module is a code object by itself, here
    # all of them are linked into one library, and two modules made from one source (the f16 and the bf16 build) define
    # templates of the same name with different bodies.  The system headers come first, outside the namespace.
    system = sorted(set(h for fn in os.listdir(KERNELS) for h in re.findall(r"^#include <(.*)>", open(os.path.join(KERNELS, fn)).read(), re.M)))
    text = ("".join("#include <%s>\n" % h for h in system) + "namespace cpusim_module_%s {\n" % name + '#include "%s"\n' % source
            + "".join("alignas(16) thread_local %s %s[(160 << 10) / sizeof(%s)];\n" % (t, n, t) for t, n in dynamic)
            + "".join('CPUSIM_REGISTER("%s", %s)\n' % (name, k) for k in kernels) + "}\n")
    if not os.path.exists(tu) or open(tu).read() != text:
        open(tu, "w").write(text)
    obj = os.path.join(out_dir, "mod_%s.o" % name)
    return obj, compile_if_stale(cxx, flags, tu, obj, marked + text), len(kernels)


def build(out_dir=None, jobs=8, verbose=False, sanitize=None):
    out_dir = out_dir or os.path.join(HERE, "_build")
    os.makedirs(out_dir, exist_ok=True)
    cxx = compiler()
    if cxx is None:
        raise RuntimeError("no clang++ (the kernel sources use clang's vector extensions)")
    # the library's host objects, as its own Makefile builds them
    run(["make", "-C", CSRC, "-j%d" % jobs])
    host = [os.path.join(CSRC, "build", n + ".o") for n in HOST_OBJECTS]
    if sanitize:  # the host sources too, from source (static_scratch.hip as plain C++: its device array becomes a host array)
        flags = (["-std=c++17", "-O1", "-fPIC", "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROCM, "include")]
                 + sanitizer_flags(sanitize))
        host = []
        for n in HOST_OBJECTS:
            src = os.path.join(CSRC, "host", n + (".hip" if n == "static_scratch" else ".cpp"))
            extra = ["-x", "c++", "-include", os.path.join(HERE, "static_scratch_host.h")] if n == "static_scratch" else []
            obj = os.path.join(out_dir, "host_%s.o" % n)
            compile_if_stale(cxx, flags + extra, src, obj, run([cxx] + flags + extra + ["-E", "-P", src]))
            host.append(obj)
    mods = modules()
    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        futures = [pool.submit(build_module, cxx, out_dir, *m, sanitize) for m in mods]
        for (name, _, _), f in zip(mods, futures):
            obj, rebuilt, count = f.result()
            if verbose:
                print("%-24s %3d kernels%s" % (name, count, "  (compiled)" if rebuilt else ""), flush=True)
            objs.append(obj)
    table = os.path.join(out_dir, "sim_modules.cpp")
    text = ('extern "C" {\nstruct EmbeddedModule { const char *name; const unsigned char *begin, *end; };\n'
            "extern const EmbeddedModule ophip_embedded_modules[] = {\n"
            + "".join('    {"%s", (const unsigned char *)"%s", nullptr},\n' % (n, n) for n, _, _ in mods)
            + "};\nextern const unsigned ophip_embedded_module_count = %d;\n}\n" % len(mods))
    if not os.path.exists(table) or open(table).read() != text:
        open(table, "w").write(text)
    host_flags = ["-std=c++20", "-O1", "-g", "-fPIC", "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(ROCM, "include"), "-I", HERE] + sanitizer_flags(sanitize)
    runtime_src = os.path.join(HERE, "sim_runtime.cpp")
    runtime_text = open(runtime_src).read() + open(os.path.join(HERE, "cpusim_core.h")).read()
    compile_if_stale(cxx, host_flags, runtime_src, os.path.join(out_dir, "sim_runtime.o"), runtime_text)
    compile_if_stale(cxx, host_flags, table, os.path.join(out_dir, "sim_modules.o"), text)
    lib = os.path.join(out_dir, "libophip_cpusim.so")
    rpath = []
    if sanitize:  # where the sanitizer's shared runtime lives
        probe = run([cxx, "-print-file-name=libclang_rt.ubsan_standalone-x86_64.so"]).strip()
        if os.path.isabs(probe):
            rpath = ["-Wl,-rpath," + os.path.dirname(os.path.realpath(probe))]
    run([cxx, "-shared", "-o", lib] + sanitizer_flags(sanitize) + rpath + host + objs
        + [os.path.join(out_dir, "sim_runtime.o"), os.path.join(out_dir, "sim_modules.o"), "-lpthread"])
    return lib


if __name__ == "__main__":
    print(build(sys.argv[1] if len(sys.argv) > 1 else None, verbose=True, sanitize=sys.argv[2] if len(sys.argv) > 2 else None))
