"""Builds libnoeira_qlinear.so (hand-written HIP for gfx950) in-tree.

    python -m noeira_amd.build            # rebuild what changed
    python -m noeira_amd.build --force

hipcc cross-compiles without a GPU.  The library is written next to this file
so that it travels with the source tree and is found by noeira_amd._lib.
Follows the reference's shim build (scripts/build_serial.sh:27-40): -fPIC,
-shared and -Wl,--no-undefined so a missing symbol is a link error here, not
an abort at the first dlopen.
"""
from __future__ import annotations

import argparse
import concurrent.futures as cf
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "csrc", "_obj")
LIB = os.path.join(HERE, "libnoeira_qlinear.so")
ROOT = os.path.dirname(HERE)

SOURCES = ["nq_api.hip", "nq_q4_0.hip", "nq_gemv.hip", "nq_quant.hip", "nq_gemm8.hip", "nq_gemm_a16.hip", "nq_mlp.hip", "nq_gemv_m1.hip", "nq_gemv_fp8.hip", "nq_gptq.hip", "nq_lora.hip", "nq_gemv_row4.hip", "nq_gemv_row8.hip", "nq_gemv_split.hip", "nq_gemv_tile.hip", "nq_diag.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
    # packed-fp32 code generation is switched off for every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
# GPTQ's codes depend on the last bit of every sum: its sums are written as separate multiplications and
# additions, and must stay that way
EXTRA_FLAGS = {"nq_gptq.hip": ["-ffp-contract=off"]}


# Kernels that request a tile ahead with `global_load` instructions in inline assembly and wait for it with an explicit
# `s_waitcnt`: the compiler takes the registers those loads write for valid from the load on, so a spill (or a copy made
# to free a register) between request and wait would store what has not arrived yet.  Their register budgets are
# chosen so that none is needed; the build refuses an object in which one of them uses scratch memory.
NO_SPILL = {"nq_gemv_tile.hip": ("gemv_tile4i_kernel", "gemv_tile4_rows_kernel", "gemv_tile8_rows_kernel"),
            "nq_gemv_fp8.hip": ("tile8_kernel",)}
# The large-tile GEMM is held to nearly the same rule for its speed: 256 accumulators per lane leave its epilogue a
# tight budget, and a variant that spilled there has cost 60 % of the call before.  One or two values parked in scratch
# memory ahead of the K loop and fetched back in the epilogue are tolerated (SPEED_SCRATCH_BYTES per lane); the K loop
# itself must stay free of scratch instructions and of register copies, which is checked on the assembly.
NO_SPILL_FOR_SPEED = {"nq_gemm8.hip": ("gemm8_kernel",)}
SPEED_SCRATCH_BYTES = 16


def _spilling_kernels(remarks: str, names, allow_bytes: int = 0) -> list:
    """From the compiler's kernel-resource-usage remarks: the kernels among `names` with scratch memory or spills
    (more than `allow_bytes` of scratch per lane)."""
    out, cur = [], None
    for l in remarks.splitlines():
        m = re.search(r"remark: Function Name: (\S+)", l)
        if m:
            cur = m.group(1) if any(n in m.group(1) for n in names) else None
            continue
        m = re.search(r"remark:\s+(ScratchSize \[bytes/lane\]|SGPRs Spill|VGPRs Spill): (\d+)", l)
        if m and cur and m.group(1) != "SGPRs Spill" and cur not in out:
            limit = allow_bytes if m.group(1).startswith("ScratchSize") else allow_bytes // 4
            if int(m.group(2)) > limit:
                out.append(cur)
    return out


# Straight-line prefetches marked in the source: loads in inline assembly whose text ends in `; pf`, waited for by
# an `s_waitcnt ... ; pfw`.  Between the two no instruction may name a register such a load writes (a copy or a
# reuse there would take what has not arrived yet): checked on the kernels' assembly.
PREFETCH_MARKED = ("nq_gemv_fp8.hip",)
# Prefetches across a loop's back edge, two register slots in turn (the persistent tile kernels): `; pf` loads, and an
# empty `; pfh <registers>` statement after the hand-written wait on every path.  While a slot may be in flight no
# move, accumulator copy, swap or spill may take one of its registers as a source: _inflight_violations, a may-analysis
# over the control-flow graph of the kernels' assembly.  (Established with the hipcc of ROCm 7.2.0; the check runs at
# every build, so another compiler that starts copying those registers fails the build instead of the numbers.)
INFLIGHT_MARKED = ("nq_gemv_tile.hip",)


def _early_uses_of_prefetched(asm: str) -> list:
    """(kernel, instruction) pairs that touch a `; pf` load's destination before that kernel's `; pfw` wait."""
    out = []
    parts = re.split(r"\n(_Z\S+): ; @\S*\n", asm)
    for k in range(1, len(parts), 2):
        body = parts[k + 1].split(".Lfunc_end")[0]
        if "; pf" not in body:
            continue
        regs, waited = set(), False
        for line in body.split("\n"):
            t = line.strip()
            if t.startswith("global_load") and t.endswith("; pf"):
                m = re.match(r"global_load_\w+ v(\d+|\[(\d+):(\d+)\]),", t)
                lo, hi = (int(m.group(2)), int(m.group(3))) if m.group(2) else (int(m.group(1)), int(m.group(1)))
                regs |= {"v%d" % x for x in range(lo, hi + 1)}
                continue
            if "; pfw" in t:
                waited = True
                break
            if regs and t and not t.startswith(";"):
                named = set(re.findall(r"\bv\d+\b", t))
                for a, b in re.findall(r"v\[(\d+):(\d+)\]", t):
                    named |= {"v%d" % x for x in range(int(a), int(b) + 1)}
                if named & regs:
                    out.append((parts[k], t))
        if not waited:
            out.append((parts[k], "no `; pfw` wait after the prefetch"))
    return out


_COPY_LIKE = ("v_mov_b", "v_pk_mov", "v_swap_b", "v_accvgpr_write", "v_accvgpr_mov", "scratch_store")


def _vregs(text: str) -> set:
    out = {int(a) for a in re.findall(r"\bv(\d+)\b", text)}
    for a, b in re.findall(r"\bv\[(\d+):(\d+)\]", text):
        out |= set(range(int(a), int(b) + 1))
    return out


def _inflight_violations(asm: str) -> list:
    """(kernel, instruction) pairs that name a vector register while a marked load into it may still be under way.

    Marks, written in the source's inline assembly: a load whose text ends in `; pf` puts its destination registers in
    flight; a statement `; pfh <registers>` (an empty assembly statement that follows the hand-written wait on every
    path and names the slot's registers) takes those out of flight; `; pfw` (a wait for everything) takes all out.
    Between the two the compiler must not copy or spill the registers - a copy made to free or to coalesce one would
    take what has not arrived, silently.  The check is a forward may-analysis over the kernel's control-flow graph
    (a loop whose second slot is requested in a block that stands later in the text is followed the way it runs),
    and it looks at the instructions a compiler adds unasked: moves, accumulator copies, swaps and spills.  (Branch
    conditions are not followed, so an instruction that merely computes in a slot's registers after the loop's last
    tile - where the slot was in fact never requested - is not held against the kernel.)"""
    out = []
    parts = re.split(r"\n(_Z\S+): ; @\S*\n", asm)
    for k in range(1, len(parts), 2):
        body = parts[k + 1].split(".Lfunc_end")[0]
        if "; pf" not in body:
            continue
        # ---- basic blocks
        blocks, cur, label_of = [[]], 0, {}
        for raw in body.split("\n"):
            t = raw.strip()
            m = re.match(r"(\.LBB\d+_\d+):", t)
            if m:
                if blocks[-1]:
                    blocks.append([])
                label_of[m.group(1)] = len(blocks) - 1
                continue
            if not t or t.startswith(".") or (t.startswith(";") and not t.startswith("; pfh") and "pfw" not in t):
                continue
            blocks[-1].append(t)
            if re.match(r"s_(c?branch\w*|endpgm|setpc)", t):
                blocks.append([])
        succ = []
        for i, b in enumerate(blocks):
            s_ = []
            last = b[-1] if b else ""
            m = re.match(r"s_(c?branch\w*)\s+(\.LBB\d+_\d+)", last)
            if m:
                if m.group(2) in label_of:
                    s_.append(label_of[m.group(2)])
                if m.group(1) != "branch" and i + 1 < len(blocks):
                    s_.append(i + 1)
            elif not last.startswith("s_endpgm") and i + 1 < len(blocks):
                s_.append(i + 1)
            succ.append(s_)
        # ---- fixpoint
        IN = [set() for _ in blocks]
        work = list(range(len(blocks)))
        bad = {}
        while work:
            i = work.pop(0)
            live = set(IN[i])
            for t in blocks[i]:
                if t.startswith("; pfh"):
                    live -= _vregs(t)
                    continue
                if "pfw" in t:
                    live = set()
                    continue
                if t.endswith("; pf"):
                    live |= _vregs(t.partition(",")[0])
                    continue
                # what the compiler inserts on its own where registers are short or values meet: copies and spills
                if live and t.startswith(_COPY_LIKE):
                    src = t if t.startswith("scratch_store") else t.partition(",")[2]
                    if _vregs(src) & live:
                        bad[(i, t)] = True
            for j in succ[i]:
                if not live <= IN[j]:
                    IN[j] |= live
                    if j not in work:
                        work.append(j)
        out += [(parts[k], t) for (_, t) in bad]
    return out


def _scratch_between_mfmas(asm: str, names) -> list:
    """Kernels among `names` with a scratch access or a register copy between their first and last v_mfma instruction.
    (The K loop's fragment reads are inline assembly whose registers the compiler takes for valid from the read on: a
    copy made between a read and its hand-written wait would take what has not arrived.  The loop as built holds no
    vector move at all, which is what this keeps true.)"""
    out = []
    parts = re.split(r"\n(_Z\S+): ; @\S*\n", asm)
    for k in range(1, len(parts), 2):
        if not any(n in parts[k] for n in names):
            continue
        lines = parts[k + 1].split(".Lfunc_end")[0].split("\n")
        mf = [i for i, l in enumerate(lines) if l.strip().startswith("v_mfma")]
        if mf and any("scratch_" in l or l.strip().startswith(("v_mov_b", "v_accvgpr_", "v_swap_b")) for l in lines[mf[0]:mf[-1] + 1]):
            out.append(parts[k])
    return out


def _deps():
    hs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    hs.append(os.path.join(ROOT, "include", "noeira_qlinear.h"))
    return hs


def _compile(src: str, force: bool) -> str:
    obj = os.path.join(OBJ, src.replace(".hip", ".o"))
    path = os.path.join(CSRC, src)
    newest = max(os.path.getmtime(p) for p in [path] + _deps())
    if not force and os.path.exists(obj) and os.path.getmtime(obj) >= newest:
        return obj
    guarded = NO_SPILL.get(src) or NO_SPILL_FOR_SPEED.get(src)
    cmd = [HIPCC] + FLAGS + EXTRA_FLAGS.get(src, []) + (["-Rpass-analysis=kernel-resource-usage"] if guarded else []) + ["-c", path, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stdout}\n{r.stderr}")
    err = r.stderr
    if guarded:
        spilled = _spilling_kernels(err, guarded, 0 if src in NO_SPILL else SPEED_SCRATCH_BYTES)
        err = "\n".join(l for l in err.splitlines() if "kernel-resource-usage" not in l and not re.match(r"^\s+(\d+ \||\|)", l))
        if spilled:
            os.remove(obj)
            raise RuntimeError(f"{src}: kernels that keep loads under way in registers, or whose register budget is tuned, "
                               f"must not spill: {spilled}")
    if src in NO_SPILL_FOR_SPEED:
        cmd = [HIPCC] + FLAGS + EXTRA_FLAGS.get(src, []) + ["--cuda-device-only", "-S", path, "-o", obj + ".s"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc -S failed on {src}:\n{r.stdout}\n{r.stderr}")
        with open(obj + ".s") as f:
            inside = _scratch_between_mfmas(f.read(), NO_SPILL_FOR_SPEED[src])
        os.remove(obj + ".s")
        if inside:
            os.remove(obj)
            raise RuntimeError(f"{src}: scratch memory is accessed, or a register copied, between the first and the last MFMA of {inside}")
    if src in PREFETCH_MARKED or src in INFLIGHT_MARKED:
        cmd = [HIPCC] + FLAGS + EXTRA_FLAGS.get(src, []) + ["--cuda-device-only", "-S", path, "-o", obj + ".s"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc -S failed on {src}:\n{r.stdout}\n{r.stderr}")
        with open(obj + ".s") as f:
            text = f.read()
        os.remove(obj + ".s")
        early = _early_uses_of_prefetched(text) if src in PREFETCH_MARKED else []
        if src in INFLIGHT_MARKED:
            if text.count("; pfh") == 0:
                early.append((src, "no `; pfh` hand-over found: the marks are gone from the source"))
            early += _inflight_violations(text)
        if early:
            os.remove(obj)
            raise RuntimeError(f"{src}: a prefetched register is named, copied or spilled before its wait: {early[:4]}")
    warn = "\n".join(l for l in err.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if warn:
        sys.stderr.write(warn + "\n")
    return obj


def build(force: bool = False, jobs: int = 8) -> str:
    os.makedirs(OBJ, exist_ok=True)
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), SOURCES))
    if force or not os.path.exists(LIB) or any(os.path.getmtime(o) > os.path.getmtime(LIB) for o in objs):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs + ["-Wl,--no-undefined"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    a = ap.parse_args()
    print(build(force=a.force))
