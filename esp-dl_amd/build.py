"""Builds the gfx950 libraries of this package in-tree with hipcc.

  python esp-dl_amd/build.py            # libespdl_hip.so (kernels + C ABI)

The GPU box runs the prebuilt .so files that travel with the tree; nothing is compiled there.
"""
import concurrent.futures
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
OBJ_DIR = os.path.join(HERE, "build")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
HIP_FLAGS = ["--offload-arch=" + ARCH, "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             # the float-defined operators (pooling, requantize, table builders) round every product to float
             # before the next operation, as the reference's C code does: no fused multiply-add
             "-ffp-contract=off",
             # keep MFMA accumulators in ordinary VGPRs: no v_accvgpr_read/write around the epilogue
             "-mllvm", "-amdgpu-mfma-vgpr-form=1"]

KERNEL_SOURCES = ["conv2d_s8_mfma.hip", "conv2d_s8_mfma_vec16.hip", "conv2d_s8_mfma_point.hip",
                  "conv2d_s8_mfma_rowseg.hip", "conv2d_s8_mfma_gather.hip", "depthwise_s8.hip", "depthwise_s8_mfma.hip", "depthwise_s8_lds.hip",
                  "conv2d_s8_pwgemm.hip", "conv2d_s8_tiled.hip", "conv2d_s8_stem.hip", "mbconv_s8_fused.hip", "mbconv_s8_staged.hip", "mbconv_s8_wave.hip", "mbconv_s8_group.hip", "conv_s16.hip", "conv_s16_mfma.hip", "elementwise_s8.hip", "elementwise_s16.hip", "layout_ops.hip", "max_pool_s8.hip", "attention_ops.hip", "espdl_hip_api.hip"]


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in r.stderr.splitlines() if noise not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s\n%s" % (" ".join(cmd), r.stdout, err))
    return err


def _compile(src, extra=()):
    obj = os.path.join(OBJ_DIR, os.path.basename(src) + ".o")
    if os.path.basename(src) in CHECKED_ASM:
        extra = (*extra, "-save-temps=obj")
    warn = _run([HIPCC, *HIP_FLAGS, *extra, "-c", src, "-o", obj])
    if os.path.basename(src) in CHECKED_ASM:
        stem = os.path.splitext(os.path.basename(src))[0]
        CHECKED_ASM[os.path.basename(src)](os.path.join(OBJ_DIR, stem + "-hip-amdgcn-amd-amdhsa-%s.s" % ARCH))
    return obj, warn


def _vgprs(text):
    """Vector registers an instruction line names (vN and v[a:b])."""
    text = text.split(";")[0]
    regs = set()
    for a, b in re.findall(r"\bv\[(\d+):(\d+)\]", text):
        regs.update(range(int(a), int(b) + 1))
    regs.update(int(a) for a in re.findall(r"\bv(\d+)\b", text))
    return regs


def check_hand_waited_loads(asm_path, kernel, expected_regs):
    """conv2d_s8_tiled.hip and depthwise_s8_lds.hip load the pieces of the next input patch with buffer loads
    written as asm statements and wait for them by hand, so the compiler does not know that the destination
    registers are in flight.  This reads the generated code of every instance of `kernel` and fails the build
    unless
      * the instance has no vector register spills, and
      * from the first load into a piece register to the end of the instance that register is named only by the
        loads of the piece, by the LDS write of the piece (as data) and by the instructions shortly in front of
        a load that compute its address in the load's own destination (the piece in it was written to LDS before).
    `expected_regs`: piece registers an instance with such loads must have (instances without any are skipped:
    builds of the kernel that fetch their input another way).
    """
    lines = open(asm_path).read().splitlines()
    starts = [i for i, l in enumerate(lines) if re.match(r"^_ZN5espdl\S*%s\S*:" % kernel, l)]
    if not starts:
        raise RuntimeError("%s: no %s in the generated code" % (asm_path, kernel))
    problems = []
    checked = 0
    for st in starts:
        name = lines[st].split(":")[0]
        end = next(i for i in range(st, len(lines)) if "s_endpgm" in lines[i])
        body = lines[st:end]
        loads, first = {}, {}
        for i, l in enumerate(body):
            m = re.search(r"buffer_load_dwordx4 v\[(\d+):(\d+)\], v(\d+)", l)
            if m:
                loads[i] = set(range(int(m.group(1)), int(m.group(2)) + 1))
                for r in loads[i]:
                    first.setdefault(r, i)
        if not first:
            continue
        checked += 1
        meta = "\n".join(lines[next(i for i, l in enumerate(lines) if ".name:" in l and name in l):][:12])
        m = re.search(r"\.vgpr_spill_count:\s*(\d+)", meta)
        if m is None or int(m.group(1)) != 0:
            problems.append("%s: vector register spills (%s)" % (name, m.group(1) if m else "count not found"))
        if len(first) != expected_regs:
            problems.append("%s: %d piece registers, expected %d" % (name, len(first), expected_regs))
        load_lines = sorted(loads)
        for i, l in enumerate(body):
            if not l.startswith("\t") or l.lstrip().startswith((";", ".")):
                continue
            named = {r for r in _vgprs(l) if r in first and i > first[r]}
            if not named:
                continue
            op = l.split()[0]
            if op == "buffer_load_dwordx4":
                continue
            if op == "ds_write_b128":
                m = re.search(r"ds_write_b128 v(\d+), v\[(\d+):(\d+)\]", l)
                if m and int(m.group(1)) not in named:
                    continue
            # address arithmetic in the destination of a load that follows within eighty lines
            ahead = [j for j in load_lines if i < j <= i + 80]
            if ahead and all(any(r in loads[j] for j in ahead) for r in named):
                continue
            problems.append("%s line %d touches a piece register: %s" % (os.path.basename(asm_path), st + i + 1, l.strip()))
    if not checked:
        problems.append("no instance of %s has hand-waited loads" % kernel)
    if problems:
        raise RuntimeError("%s: generated code breaks what the hand-placed waits assume:\n  %s"
                           % (os.path.basename(asm_path), "\n  ".join(problems[:20])))


def check_m0_only_for_lds_copies(asm_path):
    """The copies from memory straight into LDS (`buffer_load ... lds`) take their LDS address from m0, which the
    kernel source writes by hand and the compiler knows nothing about: the generated code must not use m0 for
    anything of its own (indexed register moves, for one), or a copy in flight would land somewhere else."""
    problems = []
    copies = 0
    for n, l in enumerate(open(asm_path), 1):
        code = l.split(";")[0]
        if re.search(r"\bbuffer_load_dwordx4\b.*\blds\b", code):
            copies += 1
        if re.search(r"\bm0\b", code) and not re.match(r"\s*s_mov_b32 m0, s\d+\s*$", code):
            problems.append("line %d: %s" % (n, code.strip()))
    if not copies:
        problems.append("no copy into LDS found")
    if problems:
        raise RuntimeError("%s: m0 is used by more than the hand-written LDS copies:\n  %s"
                           % (os.path.basename(asm_path), "\n  ".join(problems[:20])))


CHECKED_ASM = {
    "mbconv_s8_wave.hip": check_m0_only_for_lds_copies,
    "conv2d_s8_tiled.hip": lambda path: check_hand_waited_loads(path, "conv2d_s8_tiled_kernel", 32),
    "depthwise_s8_lds.hip": lambda path: check_hand_waited_loads(path, "depthwise_s8_lds_kernel", 20),
}


def build_kernels(verbose=True):
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    srcs = [os.path.join(CSRC, s) for s in KERNEL_SOURCES]
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        results = list(pool.map(_compile, srcs))
    for (obj, warn), src in zip(results, srcs):
        if warn.strip() and verbose:
            print("[%s]\n%s" % (os.path.basename(src), warn), file=sys.stderr)
    out = os.path.join(LIB_DIR, "libespdl_hip.so")
    _run([HIPCC, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", out, *[o for o, _ in results]])
    return out


DL_DIR = os.path.join(HERE, "dl")
DL_SOURCES = ["dl_tensor_base.cpp", "fbs_model.cpp", "fbs_loader.cpp", "dl_model_context.cpp", "dl_module_base.cpp", "dl_model_base.cpp",
              "espdl_model_capi.cpp"]
INCLUDE_DIR = os.path.join(os.path.dirname(HERE), "include")


def build_host_layer(verbose=True):
    """libespdl_dl.so: the C++ `dl::` host layer (TensorBase, Module, Model) + its C handle API."""
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    inc = ["-I" + os.path.join(DL_DIR, "include"), "-I" + INCLUDE_DIR]
    srcs = [os.path.join(DL_DIR, "src", s) for s in DL_SOURCES]

    def comp(src):
        obj = os.path.join(OBJ_DIR, os.path.basename(src) + ".o")
        warn = _run([HIPCC, "-x", "hip", "--offload-arch=" + ARCH, "-O2", "-fPIC", "-std=c++17", "-Wall",
                     "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", *inc, "-c", src, "-o", obj])
        return obj, warn

    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        results = list(pool.map(comp, srcs))
    for (obj, warn), src in zip(results, srcs):
        if warn.strip() and verbose:
            print("[%s]\n%s" % (os.path.basename(src), warn), file=sys.stderr)
    out = os.path.join(LIB_DIR, "libespdl_dl.so")
    _run([HIPCC, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", out, *[o for o, _ in results],
          "-L" + LIB_DIR, "-lespdl_hip", "-Wl,-rpath,$ORIGIN"])
    return out


def build_api_check(verbose=True):
    """lib/espdl_api_check and lib/espdl_module_api_check: small C++ programs written against the host
    layer's public headers (tests/cpp/*.cpp); the tests run them."""
    outs = []
    for stem in ("api_check", "module_api_check"):
        src = os.path.join(os.path.dirname(HERE), "tests", "cpp", stem + ".cpp")
        out = os.path.join(LIB_DIR, "espdl_" + stem)
        warn = _run([HIPCC, "-x", "hip", "--offload-arch=" + ARCH, "-O1", "-std=c++17", "-Wall",
                     "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                     "-I" + os.path.join(DL_DIR, "include"), "-I" + INCLUDE_DIR, src, "-o", out,
                     "-L" + LIB_DIR, "-lespdl_dl", "-lespdl_hip", "-Wl,-rpath,$ORIGIN"])
        if warn.strip() and verbose:
            print("[%s.cpp]\n%s" % (stem, warn), file=sys.stderr)
        outs.append(out)
    return outs


def build_all(verbose=True):
    return [build_kernels(verbose), build_host_layer(verbose), *build_api_check(verbose)]


if __name__ == "__main__":
    for lib in build_all():
        print("built", lib)
