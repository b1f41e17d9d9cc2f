"""Builds the native libraries of the package in-tree (no GPU needed: hipcc cross-compiles gfx950).

  nart_amd/lib/libhipq.so             HIP kernels + their C ABI (include/hipq.h)
  nart_amd/lib/libart.so              the minimal host core implementing the art C API (include/art/)
  nart_amd/lib/libart_module_hip.so   the `hip` case module (exports hip_module_tp)

Usage: python -m nart_amd.build [--force]
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "lib")
INC = os.path.join(ROOT, "include")

ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HIPCC = os.environ.get("HIPCC", os.path.join(ROCM, "bin", "hipcc"))
# packed-fp32 instructions are switched off on purpose (they have produced wrong results on this pool)
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function",
             # MFMA accumulators live in ordinary VGPRs: the epilogue reads them without v_accvgpr_read round trips
             "-mllvm", "-amdgpu-mfma-vgpr-form"]


def _run(cmd):
    print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def _newer(target, sources):
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(s) <= t for s in sources)


def _glob(sub, exts):
    d = os.path.join(CSRC, sub)
    if not os.path.isdir(d):
        return []
    return sorted(os.path.join(d, f) for f in os.listdir(d) if f.endswith(exts))


def build_hipq(force=False):
    srcs = _glob("hipq", (".hip", ".cpp"))
    deps = srcs + _glob("hipq", (".h",)) + [os.path.join(INC, "hipq.h")]
    out = os.path.join(LIB, "libhipq.so")
    if not force and _newer(out, deps):
        return out
    os.makedirs(LIB, exist_ok=True)
    objs, usage = [], {}

    headers = [d for d in deps if d.endswith(".h")]

    def compile_one(s):
        import json
        o = os.path.join(LIB, "obj_hipq_" + os.path.basename(s) + ".o")
        u = o + ".usage.json"  # the resource remarks of this translation unit, kept beside its object
        if not force and _newer(o, [s] + headers) and os.path.exists(u):
            with open(u) as f:
                return o, json.load(f)
        lang = ["-x", "hip"] if s.endswith(".hip") else []
        cmd = [HIPCC] + HIP_FLAGS + ["-I" + INC, "-I" + os.path.join(CSRC, "hipq"), "-c"] + lang + [s, "-o", o]
        usage = {}
        if s.endswith(".hip"):
            usage = _compile_with_usage(cmd)
        else:
            _run(cmd)
        with open(u, "w") as f:
            json.dump(usage, f)
        return o, usage
    from concurrent.futures import ThreadPoolExecutor
    with ThreadPoolExecutor(max_workers=4) as pool:  # the translation units are independent; the largest takes minutes
        for o, u in pool.map(compile_one, srcs):
            objs.append(o)
            usage.update(u)
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out] + objs)
    import json
    with open(os.path.join(LIB, "kernel_resources.json"), "w") as f:
        json.dump(usage, f, indent=0, sort_keys=True)
    return out


def _compile_with_usage(cmd):
    """Compile one HIP source with the compiler's per-kernel resource remarks switched on and return
    {mangled kernel name: {"vgprs", "scratch", "lds", "occupancy"}}.  A kernel that uses scratch memory (a register
    array that the optimiser could not keep in registers, or spills) fails the build: every kernel here is written to
    live in registers, and one careless edit of a shared epilogue has cost the largest tiles a factor of three."""
    import re
    cmd = cmd + ["-Rpass-analysis=kernel-resource-usage"]
    print(" ".join(cmd), flush=True)
    p = subprocess.run(cmd, stderr=subprocess.PIPE, text=True)
    keep = [ln for ln in p.stderr.splitlines() if "-Rpass-analysis=kernel-resource-usage" not in ln
            and "not a recognized feature" not in ln]
    if keep:
        print("\n".join(keep), file=sys.stderr, flush=True)
    if p.returncode != 0:
        raise subprocess.CalledProcessError(p.returncode, cmd)
    usage, cur = {}, None
    keys = {"VGPRs": "vgprs", "ScratchSize [bytes/lane]": "scratch", "LDS Size [bytes/block]": "lds",
            "Occupancy [waves/SIMD]": "occupancy"}
    for ln in p.stderr.splitlines():
        m = re.search(r"remark:\s+Function Name: (\S+)", ln)
        if m:
            cur = usage.setdefault(m.group(1), {})
            continue
        m = re.search(r"remark:\s+([A-Za-z /\[\]]+): (\d+)", ln)
        if m and cur is not None and m.group(1).strip() in keys:
            cur[keys[m.group(1).strip()]] = int(m.group(2))
    bad = sorted(k for k, v in usage.items() if v.get("scratch", 0) > 0)
    if bad:
        raise RuntimeError("kernels that use scratch memory (bytes per lane): "
                           + ", ".join("%s=%d" % (k, usage[k]["scratch"]) for k in bad))
    return usage


def build_art(force=False):
    outs = []
    core_src = _glob("core", (".c", ".cpp"))
    if core_src:
        out = os.path.join(LIB, "libart.so")
        deps = core_src + _glob("core", (".h",)) + [os.path.join(INC, "art", f) for f in os.listdir(os.path.join(INC, "art"))]
        if force or not _newer(out, deps):
            _run(["gcc", "-O2", "-std=gnu11", "-fPIC", "-shared", "-Wall", "-fvisibility=hidden", "-I" + INC,
                  "-I" + os.path.join(CSRC, "core"), "-o", out] + core_src + ["-lm"])
        outs.append(out)
    outs += build_module(force)
    return outs


def build_module(force=False, nart_tree=None, out_name="libart_module_hip.so"):
    """The `hip` case module.  nart_tree: path of a NART checkout — then the module is compiled against the
    runtime's own headers instead of include/art/art.h (how a NART maintainer would build it)."""
    mod_src = _glob("module", (".cpp", ".c"))
    if not mod_src:
        return []
    out = os.path.join(LIB, out_name)
    deps = mod_src + _glob("module", (".h",)) + [os.path.join(INC, "hipq.h"), os.path.join(INC, "art", "art.h")]
    if not force and _newer(out, deps):
        return [out]
    inc = ["-I" + INC, "-I" + os.path.join(CSRC, "module")]
    if nart_tree:
        art = os.path.join(nart_tree, "art")
        inc += ["-DNART_HIP_USE_NART_HEADERS", "-DART_CONSTRAINT_WITH_NAME", "-DNART_LOG_LEVEL=1",
                "-I" + os.path.join(art, "include"), "-I" + os.path.join(art, "modules", "quant", "include")]
    objs = []
    for s in mod_src:
        o = os.path.join(LIB, "obj_%s_%s.o" % (out_name.split(".")[0], os.path.basename(s)))
        if s.endswith(".c"):
            _run(["gcc", "-O2", "-std=gnu11", "-fPIC", "-Wall"] + inc + ["-c", s, "-o", o])
        else:
            # host-only C++ (no device code in the module): the HIP runtime API through its AMD platform headers
            _run(["g++", "-O2", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function", "-D__HIP_PLATFORM_AMD__",
                  "-I" + os.path.join(ROCM, "include")] + inc + ["-c", s, "-o", o])
        objs.append(o)
    _run(["g++", "-shared", "-fPIC", "-o", out] + objs + ["-L" + LIB, "-lhipq", "-L" + os.path.join(ROCM, "lib"),
                                                          "-lamdhip64", "-Wl,-rpath,$ORIGIN"])
    return [out]


def build_tools(force=False):
    """nart_promark, the command-line runner (counterpart of the reference's tools/promark.cpp); finds libart.so and
    the case modules next to itself."""
    src = _glob("tools", (".cpp",))
    out = os.path.join(LIB, "nart_promark")
    if src and (force or not _newer(out, src + [os.path.join(INC, "art", "art.h")])):
        _run(["g++", "-O2", "-std=c++17", "-Wall", "-I" + INC, "-o", out] + src +
             ["-L" + LIB, "-lart", "-ldl", "-Wl,--disable-new-dtags", "-Wl,-rpath,$ORIGIN"])
    return [out] if src else []


def build_all(force=False):
    return [build_hipq(force)] + build_art(force) + build_tools(force)


if __name__ == "__main__":
    print("\n".join(build_all("--force" in sys.argv)))
