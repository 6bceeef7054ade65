"""What each part of the main kernel costs: builds copies of the library with parts of spmm_bitmap_rows switched off
and times them on the GPU, each against the complete kernel in the same run.

    python -m spmspm_amd.ablate [--shape 28672x7168] [--n 16] [--sparsity 0.7] [--split-k 0] [--steps 500]

The kernel source is not written for this: the variants are made by textual patches of csrc/spmm_kernels.hiph into a
temporary directory (a patch that no longer applies is an error), compiled with the library's own flags and called
through the same C ABI.  A variant computes wrong sums by construction; only its time is read.  Registers whose
loads are removed are passed through an empty asm statement so that the compiler keeps everything downstream.

Variants (the complete kernel is always the first and the last line):
  no X loads            the two X operand loads per tile are not issued
  X from four k blocks  X operands always come from k blocks 0..3 (cache hits): the address path without the L2 traffic
  no epilogue           no cross-wave sum, no partial-sum stores
  no partial stores     the cross-wave sum runs, nothing is stored
  loads only            no LDS staging, no decode: global loads, waits and the epilogue
  loads only, no X
  decode only           no global loads of values, bitmaps or X: LDS staging, decode and the epilogue on stale registers
  decode only, no epilogue
  structure only        neither loads nor staging nor decode: launch, offsets, loop and epilogue
  windows as two aligned 8-byte reads + select
                        a different decode, not a removal: half of a tile's 16 window fetches cost half the LDS
                        cycles (6.2 against 12.9 per fetch) and four more VALU instructions each
"""
import argparse
import ctypes
import os
import shutil
import subprocess
import sys
import tempfile

import numpy as np

from . import build

PATCHES = [
    # (old, new): applied once each, in order
    ("#pragma once",
     "#pragma once\n" + "".join(f"#ifndef {m}\n#define {m} 0\n#endif\n" for m in
                                ("ABL_NOX", "ABL_XFIXED", "ABL_NOVAL", "ABL_NOBM", "ABL_NOSTAGE", "ABL_NODECODE",
                                 "ABL_NOEPI", "ABL_NOSTORE", "ABL_B64"))),
    ("namespace spmm {\n",
     "namespace spmm {\n"
     "__device__ __forceinline__ void abl_touch(uint4& v) { asm volatile(\"\" : \"+v\"(v.x), \"+v\"(v.y), \"+v\"(v.z), \"+v\"(v.w)); }\n"
     "__device__ __forceinline__ void abl_touch(uint2& v) { asm volatile(\"\" : \"+v\"(v.x), \"+v\"(v.y)); }\n"
     "template <typename T> __device__ __forceinline__ void abl_touch16(T& h) { uint4 u = __builtin_bit_cast(uint4, h); abl_touch(u); h = __builtin_bit_cast(T, u); }\n"),
    ("    uint4 pv0, pv1, pv2, pv3, pv4, pv5;",
     "    uint4 pv0 = {}, pv1 = {}, pv2 = {}, pv3 = {}, pv4 = {}, pv5 = {};"),
    ("    uint2 pb;  ", "    uint2 pb = {};"),
    ("    half8 pxA[NT][2], pxB[NT][2];      ", "    half8 pxA[NT][2] = {}, pxB[NT][2] = {};"),
    ("    if ((C_) * 512 < p_nnz) { /* wave-uniform; lanes past the end re-read the last chunk */",
     "    if (ABL_NOVAL) abl_touch(pv##C_); else if ((C_) * 512 < p_nnz) {"),
    ("            const uint16_t* xp_ = xrow + (size_t)nt * 16 * K + (size_t)(KB) * 64;      ",
     "            const uint16_t* xp_ = xrow + (size_t)nt * 16 * K + (size_t)(ABL_XFIXED ? ((KB) & 3) : (KB)) * 64;"),
    ("            px##XS[nt][0]       = *reinterpret_cast<const half8*>(xp_);",
     "            if (ABL_NOX) { abl_touch16(px##XS[nt][0]); abl_touch16(px##XS[nt][1]); continue; } px##XS[nt][0] = *reinterpret_cast<const half8*>(xp_);"),
    ("        pb = reinterpret_cast<const uint2*>(bitmaps + (size_t)(G) * 64)[lane];",
     "        if (ABL_NOBM) abl_touch(pb); else pb = reinterpret_cast<const uint2*>(bitmaps + (size_t)(G) * 64)[lane];"),
    ("#define SPMM_TILE_STAGE()                                                                                         \\\n    do {",
     "#define SPMM_TILE_STAGE()                                                                                         \\\n    do {"
     " if (ABL_NOSTAGE) { asm volatile(\"s_waitcnt vmcnt(0)\"); abl_touch(pv0); abl_touch(pv1); abl_touch(pv2); abl_touch(pv3); abl_touch(pv4); abl_touch(pv5); abl_touch(pb); break; }"),
    ("#define SPMM_TILE_DECODE(XS)                                                                                      \\\n    do {",
     "#define SPMM_TILE_DECODE(XS)                                                                                      \\\n    do {"
     " if (ABL_NODECODE) { abl_touch16(px##XS[0][0]); abl_touch16(px##XS[0][1]); break; }"),
    ("    // ---- cross-wave sum through LDS.",
     "    if (ABL_NOEPI) { if (acc[0][0][0] == 12345.f) static_cast<float*>(out)[0] = 1.f; return; }\n"
     "    // ---- cross-wave sum through LDS."),
    ("            __builtin_nontemporal_store(s4,", "            if (!ABL_NOSTORE || s4[0] == 12345.f) __builtin_nontemporal_store(s4,"),
    # ABL_B64 = bit mask over a tile's 16 windows (bit 2*step + nibble): those windows are read as two aligned
    # 8-byte pieces and a dword select instead of three dwords.  This variant computes correct sums.
    ("        unsigned d0, d1, d2, g0, g1, g2, a0, a1;", "        unsigned d0, d1, d2, d3, g0, g1, g2, g3, a0, a1;"),
    ("        f.d0 = w0[0], f.d1 = w0[1], f.d2 = w0[2];\n        f.g0 = w1[0], f.g1 = w1[1], f.g2 = w1[2];",
     "        if ((ABL_B64 >> (2 * sigma)) & 1) { const uint2 q0 = *reinterpret_cast<const uint2*>(smem + (f.a0 & ~7u)), q1 = *reinterpret_cast<const uint2*>(smem + (f.a0 & ~7u) + 8); f.d0 = q0.x, f.d1 = q0.y, f.d2 = q1.x, f.d3 = q1.y; }\n"
     "        else { f.d0 = w0[0], f.d1 = w0[1], f.d2 = w0[2], f.d3 = 0; }\n"
     "        if ((ABL_B64 >> (2 * sigma + 1)) & 1) { const uint2 q0 = *reinterpret_cast<const uint2*>(smem + (f.a1 & ~7u)), q1 = *reinterpret_cast<const uint2*>(smem + (f.a1 & ~7u) + 8); f.g0 = q0.x, f.g1 = q0.y, f.g2 = q1.x, f.g3 = q1.y; }\n"
     "        else { f.g0 = w1[0], f.g1 = w1[1], f.g2 = w1[2], f.g3 = 0; }"),
    ("        const unsigned f0 = __builtin_amdgcn_alignbyte(cur.d1, cur.d0, cur.a0);",
     "        if ((ABL_B64 >> (2 * sigma)) & 1) { const bool u = (cur.a0 & 4u) != 0; cur.d0 = u ? cur.d1 : cur.d0, cur.d1 = u ? cur.d2 : cur.d1, cur.d2 = u ? cur.d3 : cur.d2; }\n"
     "        if ((ABL_B64 >> (2 * sigma + 1)) & 1) { const bool u = (cur.a1 & 4u) != 0; cur.g0 = u ? cur.g1 : cur.g0, cur.g1 = u ? cur.g2 : cur.g1, cur.g2 = u ? cur.g3 : cur.g2; }\n"
     "        const unsigned f0 = __builtin_amdgcn_alignbyte(cur.d1, cur.d0, cur.a0);"),
]

NOLOAD = ["-DABL_NOVAL=1", "-DABL_NOBM=1", "-DABL_NOX=1"]
VARIANTS = [
    ("complete kernel", []),
    ("no X loads", ["-DABL_NOX=1"]),
    ("X from four k blocks (cache hits)", ["-DABL_XFIXED=1"]),
    ("no epilogue", ["-DABL_NOEPI=1"]),
    ("no partial stores", ["-DABL_NOSTORE=1"]),
    ("no X loads, no epilogue", ["-DABL_NOX=1", "-DABL_NOEPI=1"]),
    ("loads only", ["-DABL_NOSTAGE=1", "-DABL_NODECODE=1"]),
    ("loads only, no X", ["-DABL_NOSTAGE=1", "-DABL_NODECODE=1", "-DABL_NOX=1"]),
    ("loads only, no epilogue", ["-DABL_NOSTAGE=1", "-DABL_NODECODE=1", "-DABL_NOEPI=1"]),
    ("decode only", NOLOAD),
    ("decode only, no epilogue", NOLOAD + ["-DABL_NOEPI=1"]),
    ("structure only", NOLOAD + ["-DABL_NOSTAGE=1", "-DABL_NODECODE=1"]),
    ("structure only, no epilogue", NOLOAD + ["-DABL_NOSTAGE=1", "-DABL_NODECODE=1", "-DABL_NOEPI=1"]),
    # (with all 16 windows in that form this patched source needs more than the 128 registers and spills)
    ("the 8 low-nibble windows as two aligned 8-byte reads + select (correct sums)", ["-DABL_B64=0x5555u"]),
    ("the 8 high-nibble windows in that form (correct sums)", ["-DABL_B64=0xaaaau"]),
    ("complete kernel (again)", []),
]


def patched_sources(workdir):
    """Copies csrc/ into workdir with spmm_kernels.hiph patched."""
    for f in os.listdir(build.CSRC):
        shutil.copy(os.path.join(build.CSRC, f), os.path.join(workdir, f))
    path = os.path.join(workdir, "spmm_kernels.hiph")
    text = open(path).read()
    for old, new in PATCHES:
        if text.count(old) < 1:
            raise RuntimeError("ablation patch does not apply any more: " + old.splitlines()[0][:70])
        text = text.replace(old, new, 1)
    open(path, "w").write(text)


def build_variant(workdir, flags, out):
    cmd = [build.hipcc(), *build.HIPCC_FLAGS, *flags, "-I", os.path.join(build.ROOT, "include"), "-I", workdir]
    cmd += [os.path.join(workdir, s) for s in build.SOURCES] + ["-o", out, "-lpthread"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError("hipcc failed for " + " ".join(flags))
    return out


class Hip:
    def __init__(self):
        self.rt = ctypes.CDLL("libamdhip64.so")
        self.rt.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.rt.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]

    def event(self):
        e = ctypes.c_void_p()
        assert self.rt.hipEventCreate(ctypes.byref(e)) == 0
        return e

    def elapsed_ms(self, a, b):
        ms = ctypes.c_float()
        assert self.rt.hipEventElapsedTime(ctypes.byref(ms), a, b) == 0
        return ms.value


def time_library(path, torch, hip, copies, x, out, ws, M, N, K, sk, steps, warm):
    """(main kernel average us from events on its dispatches, whole call us from events around the run)."""
    L = ctypes.CDLL(path)
    L.SpMM_SplitK_API.restype = ctypes.c_int
    L.SpMM_SplitK_API.argtypes = [ctypes.c_void_p] * 6 + [ctypes.c_int] * 3 + [ctypes.c_void_p, ctypes.c_int]
    L.SpMM_TimeNextCall.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
    stream = torch.cuda.current_stream().cuda_stream

    def call(i):
        v, b, o = copies[i % len(copies)]
        err = L.SpMM_SplitK_API(stream, v.data_ptr(), b.data_ptr(), o.data_ptr(), x.data_ptr(), out.data_ptr(), M, N, K,
                                ws.data_ptr() if ws is not None else None, sk)
        assert err == 0, err

    for i in range(warm):
        call(i)
    torch.cuda.synchronize()
    g0, g1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    g0.record()
    for i in range(steps):
        call(i)
    g1.record()
    torch.cuda.synchronize()
    whole = g0.elapsed_time(g1) / steps * 1e3
    ev = [(hip.event(), hip.event()) for _ in range(steps)]
    for i in range(steps):
        L.SpMM_TimeNextCall(ev[i][0], ev[i][1])
        call(i)
    torch.cuda.synchronize()
    main = float(np.mean([hip.elapsed_ms(a, b) for a, b in ev])) * 1e3
    return main, whole


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--shape", default="28672x7168")
    ap.add_argument("--n", type=int, default=16)
    ap.add_argument("--sparsity", type=float, default=0.7)
    ap.add_argument("--split-k", type=int, default=0)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=300)
    a = ap.parse_args(argv)
    import torch

    import spmspm_amd as S
    from .synthetic import make_activations, make_weight
    M, K = (int(v) for v in a.shape.lower().split("x"))
    N = a.n
    if N >= 64 and M >= 256:
        ap.error("these patches are of spmm_bitmap_rows; N >= 64 on at least 256 rows runs on the wide kernel")
    dev = torch.device("cuda:0")
    W = make_weight(M, K, a.sparsity, seed=0, pruning="random")
    comp = S.InitSparseMatrixA_bitmap(W)
    first = S.SparseLinear(comp, device=dev)
    per_copy = 2 * first.nnz_padded + 8 * first.bitmaps.numel()
    n_copies = max(2, (768 << 20) // per_copy + 1)  # rotate over more than the last-level cache holds
    layers = [first] + [first.clone() for _ in range(n_copies - 1)]
    copies = [(l.values, l.bitmaps, l.offsets) for l in layers]
    x = torch.from_numpy(make_activations(K, N, seed=0).view(np.int16).copy()).to(dev).view(torch.float16)
    out = torch.empty((N, M), dtype=torch.float16, device=dev)
    sk = a.split_k if a.split_k > 0 else S.SpMM_SplitK_Auto(M, N, K)
    nbytes = S.SpMM_WorkspaceBytes(M, N, K, sk)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev) if nbytes else None
    hip = Hip()
    print(f"# {M}x{K}, {a.sparsity:.0%} sparse (random), N = {N}, Split_K = {sk}, {n_copies} weight copies rotated, "
          f"{a.steps} timed calls after {a.warmup}")
    print("| variant | main kernel us | whole call us |\n|---|---|---|", flush=True)
    with tempfile.TemporaryDirectory() as tmp:
        patched_sources(tmp)
        for i, (name, flags) in enumerate(VARIANTS):
            lib = build_variant(tmp, flags, os.path.join(tmp, f"ablate_{i}.so"))
            m, w = time_library(lib, torch, hip, copies, x, out, ws, M, N, K, sk, a.steps, a.warmup)
            note = ""
            if i == 0:
                ref = out.clone()
            elif "(correct sums)" in name:
                note = " C identical" if torch.equal(out.view(torch.int16), ref.view(torch.int16)) else " C DIFFERS"
            print(f"| {name}{note} | {m:.1f} | {w:.1f} |", flush=True)


if __name__ == "__main__":
    main()
