"""Compiles the HIP sources under csrc/ into warpconvnet_amd/libwcn_hip.so for gfx950."""
import glob
import os
import re
import shutil
import subprocess

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libwcn_hip.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    # packed fp32 instructions are kept out of every code object of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = "is not a recognized feature for this target"
    log = "\n".join(l for l in proc.stdout.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}): {' '.join(cmd)}\n{log}")
    return log


# Sources whose kernels issue loads in inline assembly and wait for them by count: a register the
# compiler spills (or otherwise moves) while such a load is still in flight would be overwritten
# later by the landing data.  These files must compile without any scratch memory.
NO_SCRATCH_SOURCES = ("wcn_conv_pack_f16.hip", "wcn_conv_pack_bf16.hip", "wcn_conv_pack_f32.hip")
_REMARK = "-Rpass-analysis=kernel-resource-usage"


def _extra_flags(src):
    return [_REMARK] if os.path.basename(src) in NO_SCRATCH_SOURCES else []


def _without_remarks(log):
    return "\n".join(l for l in log.splitlines() if _REMARK not in l)


def _check_no_scratch(src, log):
    if os.path.basename(src) not in NO_SCRATCH_SOURCES:
        return
    name, seen = None, 0
    for line in log.splitlines():
        if "remark: Function Name:" in line:
            name = line.split("Function Name:")[1].split("[")[0].strip()
        elif "ScratchSize [bytes/lane]:" in line or "VGPRs Spill:" in line:
            seen += 1
            value = int(line.split(":")[-1].split("[")[0].strip())
            if value != 0:
                raise RuntimeError(f"{os.path.basename(src)}: kernel {name} uses scratch memory / spills vector "
                                   f"registers ({line.split('remark:')[1].strip()}); its hand-counted loads "
                                   "make that unsafe")
    if seen == 0:
        raise RuntimeError(f"{os.path.basename(src)}: no resource-usage remarks found; cannot vouch for its kernels")


def _vgprs_in(text):
    regs = set()
    for m in re.finditer(r"v\[(\d+):(\d+)\]", text):
        regs.update(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"(?<![\w\[])v(\d+)\b", text):
        regs.add(int(m.group(1)))
    return regs


def _check_loads_not_copied(src, asm_text):
    """The destination of a written-out load must not be read or moved before a vmcnt wait: a
    copy the compiler inserts between the load and its wait (at a control-flow merge, say) would
    carry the register's old contents.  Checked on the generated code, in program-text order,
    over the copy-like instructions of the 400 lines after each such load."""
    lines = asm_text.split("\n")
    code = [l.split(";")[0].rstrip() for l in lines]
    in_asm, bad = False, []
    for i, raw in enumerate(lines):
        if "#ASMSTART" in raw:
            in_asm = True
            continue
        if "#ASMEND" in raw:
            in_asm = False
            continue
        m = re.match(r"\s*global_load_dword(x2|x4)?\s+(\S+),", code[i])
        if not (in_asm and m):
            continue
        dst = _vgprs_in(m.group(2))
        for j in range(i + 1, min(len(code), i + 400)):
            st = code[j].strip()
            if "s_endpgm" in st or ("s_waitcnt" in st and "vmcnt" in st):
                break
            ops = st.split(None, 1)
            if len(ops) > 1 and re.match(r"v_(mov|cndmask|accvgpr|perm|swap)", st) and _vgprs_in(ops[1]) & dst:
                bad.append(f"line {i + 1}: {code[i].strip()}  ->  line {j + 1}: {st}")
                break
    if bad:
        raise RuntimeError(f"{os.path.basename(src)}: the compiler moves registers that loads are still in flight "
                           "into:\n  " + "\n  ".join(bad[:10]))


def build_library(verbose: bool = False) -> str:
    """Every source file is compiled to an object of its own (in parallel), then linked."""
    from concurrent.futures import ThreadPoolExecutor
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    sources = sorted(glob.glob(os.path.join(_PKG, "csrc", "*.hip")))
    if not sources:
        raise RuntimeError("no HIP sources found under csrc/")
    objdir = os.path.join(_PKG, "build")
    os.makedirs(objdir, exist_ok=True)
    compile_flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    objects = [os.path.join(objdir, os.path.basename(src)[:-4] + ".o") for src in sources]
    cmds = [[hipcc, *compile_flags, *_extra_flags(src), "-c", "-o", obj, src]
            for src, obj in zip(sources, objects)]
    with ThreadPoolExecutor(max_workers=min(8, len(cmds))) as pool:
        logs = list(pool.map(_run, cmds))
    for src, log in zip(sources, logs):
        _check_no_scratch(src, log)
    checked = [src for src in sources if os.path.basename(src) in NO_SCRATCH_SOURCES]
    asm_paths = [os.path.join(objdir, os.path.basename(src)[:-4] + ".s") for src in checked]
    with ThreadPoolExecutor(max_workers=min(8, max(1, len(checked)))) as pool:
        list(pool.map(_run, [[hipcc, *compile_flags, "-S", "--cuda-device-only", "-o", asm, src]
                             for src, asm in zip(checked, asm_paths)]))
    for src, asm in zip(checked, asm_paths):
        with open(asm) as f:
            _check_loads_not_copied(src, f.read())
        os.remove(asm)
    logs = [_without_remarks(log) for log in logs]
    logs.append(_run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", LIB_PATH, *objects]))
    if verbose:
        for cmd in cmds:
            print(" ".join(cmd))
        text = "\n".join(l for l in logs if l.strip())
        if text:
            print(text)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
