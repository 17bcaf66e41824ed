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
# Sources whose waits are the compiler's, so that a spill is safe, but whose instances are sized to
# their register budget (waves per workgroup chosen so that nothing spills): scratch memory there is
# a slower kernel that nobody asked for, and the build says so.
NO_SPILL_SOURCES = ("wcn_conv_group.hip",)
_REMARK = "-Rpass-analysis=kernel-resource-usage"


def _extra_flags(src):
    return [_REMARK] if os.path.basename(src) in NO_SCRATCH_SOURCES + NO_SPILL_SOURCES else []


def _without_remarks(log):
    return "\n".join(l for l in log.splitlines() if _REMARK not in l)


def _check_no_scratch(src, log):
    if os.path.basename(src) not in NO_SCRATCH_SOURCES + NO_SPILL_SOURCES:
        return
    name, seen = None, 0
    for line in log.splitlines():
        if "remark: Function Name:" in line:
            name = line.split("Function Name:")[1].split("[")[0].strip()
        elif "ScratchSize [bytes/lane]:" in line or "VGPRs Spill:" in line:
            seen += 1
            value = int(line.split(":")[-1].split("[")[0].strip())
            if value != 0:
                why = ("its hand-counted loads make that unsafe" if os.path.basename(src) in NO_SCRATCH_SOURCES
                       else "its instances are meant to fit their register budget")
                raise RuntimeError(f"{os.path.basename(src)}: kernel {name} uses scratch memory / spills vector "
                                   f"registers ({line.split('remark:')[1].strip()}); {why}")
    if seen == 0:
        raise RuntimeError(f"{os.path.basename(src)}: no resource-usage remarks found; cannot vouch for its kernels")


def _vgprs_in(text):
    regs = set()
    for m in re.finditer(r"v\[(\d+):(\d+)\]", text):
        regs.update(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"(?<![\w\[])v(\d+)\b", text):
        regs.add(int(m.group(1)))
    return regs


def _loads_in_flight_touched(name, lines):
    """One kernel's listing: every use of a written-out load's destination that some path reaches
    before a wait that covers the load."""
    code = [l.split(";")[0].strip() for l in lines]
    in_asm, asm_load, labels = False, {}, {}
    for i, raw in enumerate(lines):
        if "#ASMSTART" in raw:
            in_asm = True
        elif "#ASMEND" in raw:
            in_asm = False
        else:
            m = re.match(r"global_load_dword(x2|x4)?\s+(\S+),", code[i])
            if in_asm and m:
                asm_load[i] = _vgprs_in(m.group(2))
            m = re.match(r"(\.LBB\d+_\d+):", code[i])
            if m:
                labels[m.group(1)] = i
    if not asm_load:
        return []
    n = len(code)
    load_lines, last_load = sorted(asm_load), max(asm_load)

    def successors(i):
        st = code[i]
        m = re.match(r"s_(c?)branch\w*\s+(\.LBB\d+_\d+)", st)
        if m:
            target = labels.get(m.group(2))
            nxt = [target] if target is not None else []
            # Every step issues its loads on every path, so a jump forward over some of them to a
            # place that is still among the steps is either the way out of the loop spelled as a
            # chain of tests or a path that cannot be taken: not walked.
            if target is not None and i < target <= last_load and any(i < l < target for l in load_lines):
                nxt = []
            # likewise a jump from among the steps back to before the first of them: the loop is left
            # (its condition is tested up there), not entered again
            if target is not None and target < load_lines[0] and i < last_load:
                nxt = []
            return nxt + ([i + 1] if m.group(1) and i + 1 < n else [])
        if st.startswith("s_endpgm"):
            return []
        return [i + 1] if i + 1 < n else []

    bad = []
    for start, dst in asm_load.items():
        # states: (instruction, written-out loads issued since `start`); they are issued on every path
        seen, todo, hit = set(), [(s, 0) for s in successors(start)], None
        while todo and hit is None:
            i, issued = todo.pop()
            if (i, issued) in seen:
                continue
            seen.add((i, issued))
            st = code[i]
            if i in asm_load:
                if asm_load[i] & dst:
                    continue  # the register takes its next load: this path is done
                issued = min(issued + 1, 63)
            elif st and not st.startswith((".", "#")):
                m = re.search(r"s_waitcnt.*vmcnt\((\d+)\)", st)
                if m:  # loads retire in order: all but the last N have landed
                    if int(m.group(1)) <= issued:
                        continue
                else:
                    ops = st.split(None, 1)
                    if len(ops) > 1 and _vgprs_in(ops[1]) & dst:
                        hit = f"{name}: line {start + 1}: {code[start]}  ->  line {i + 1}: {st}"
                        break
            todo.extend((s, issued) for s in successors(i))
        if hit:
            bad.append(hit)
    return bad


def _written_out_loads(lines):
    """(number of loads written out in inline assembly, whether a branch behind the last of them
    leads back to or before the first): what a kernel with a ring of such loads must show."""
    code = [l.split(";")[0].strip() for l in lines]
    in_asm, loads, labels = False, [], {}
    for i, raw in enumerate(lines):
        if "#ASMSTART" in raw:
            in_asm = True
        elif "#ASMEND" in raw:
            in_asm = False
        else:
            if in_asm and re.match(r"global_load_dword(x2|x4)?\s+\S+,", code[i]):
                loads.append(i)
            m = re.match(r"(\.LBB\d+_\d+):", code[i])
            if m:
                labels[m.group(1)] = i
    if not loads:
        return 0, False
    back = False
    for i, st in enumerate(code):
        m = re.match(r"s_c?branch\w*\s+(\.LBB\d+_\d+)", st)
        if m and i > loads[0] and labels.get(m.group(1), n_inf) <= loads[0]:
            back = True
    return len(loads), back


n_inf = 1 << 60
# Kernels that are known to keep loads in flight across their loop (by name): a listing in which
# the checker recognises none of them, or no loop around them, means the checker no longer reads
# the compiler's output (another spelling of the markers, labels or mnemonics), not that all is well.
RING_KERNELS = ("conv_fwd_pack",)


def _check_loads_not_copied(src, asm_text):
    """The destination of a written-out load must not be read, moved or overwritten before a vmcnt
    wait that covers the load: a copy the compiler inserts between the load and its wait (at a
    control-flow merge or at the loop's back edge, say) would carry the register's old contents.
    Checked on the generated code of every kernel: from each such load along every path of the
    control flow, counting the written-out loads issued since, up to a wait that covers it."""
    lines = asm_text.split("\n")
    starts = [(i, m.group(1)) for i, l in enumerate(lines) for m in [re.match(r"^(_Z\w+):", l)] if m]
    bad = []
    for n, (begin, name) in enumerate(starts):
        end = starts[n + 1][0] if n + 1 < len(starts) else len(lines)
        bad += _loads_in_flight_touched(name, lines[begin:end])
        if any(k in name for k in RING_KERNELS):
            count, loops = _written_out_loads(lines[begin:end])
            if count == 0 or not loops:
                raise RuntimeError(f"{os.path.basename(src)}: {name}: {count} written-out loads recognised, "
                                   f"loop around them {'found' if loops else 'not found'}: the listing is not "
                                   "what this check was written for, so it cannot vouch for the kernel")
    if bad:
        raise RuntimeError(f"{os.path.basename(src)}: the compiler touches registers that loads are still in flight "
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
