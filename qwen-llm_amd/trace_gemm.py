#!/usr/bin/env python3
"""Time stamps from inside the few-row Q4_K GEMM kernels (debug build -DDFLASH_TRACE): when, after the earliest
workgroup's start, a wave has its activations, reaches and passes the slab barrier, finds stage t landed, and ends.

    python qwen-llm_amd/trace_gemm.py --build            # here (hipcc cross-compiles): qwen-llm_amd/_trace/libdflash_hip_trace.so
    python qwen-llm_amd/trace_gemm.py [--n-in 5120 --n-out 17408] [--row-order]      # on the GPU

The trace library is a second build of the same sources and is loaded on its own (the product library is untouched);
the stamps (s_memrealtime + a store per stamp) slow the kernel by 10..20 %, so read them as a profile, not a duration.
"""
import argparse
import ctypes as C
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
TRACE_DIR = os.path.join(HERE, "_trace")
TRACE_LIB = os.path.join(TRACE_DIR, "libdflash_hip_trace.so")
NAMES = ["activations in registers", "at the slab barrier", "past the slab barrier", "end",
         "stage 0 landed", "stage 1 landed", "stage 2 landed", "stage 3 landed"]


def build():
    import importlib.util
    spec = importlib.util.spec_from_file_location("_b", os.path.join(HERE, "build.py"))
    b = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(b)
    os.makedirs(TRACE_DIR, exist_ok=True)
    objs, procs = [], []
    for src in b.sources():
        obj = os.path.join(TRACE_DIR, os.path.basename(src)[:-4] + ".o")
        cmd = [b.HIPCC] + [f for f in b.FLAGS if f != "-shared"] + [b.RESOURCE_FLAG, "-DDFLASH_TRACE", "-c", src, "-o", obj]
        procs.append(subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True))
        objs.append(obj)
    for p in procs:
        out, _ = p.communicate()
        if p.returncode:
            sys.exit(b.strip_remarks(out))
        # the stamps cost registers: a kernel that starts to spill with them may save a register an asm load is still
        # filling (see build.py), so such a build is refused, not run
        bad = b.check_no_scratch(out)
        if bad:
            sys.exit("the trace build spills in kernels that keep loads in flight; not usable:\n  " + "\n  ".join(bad))
    subprocess.check_call([b.HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", TRACE_LIB] + objs)
    for o in objs:
        os.remove(o)
    print(TRACE_LIB)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--build", action="store_true")
    ap.add_argument("--n-in", type=int, default=5120)
    ap.add_argument("--n-out", type=int, default=17408)
    ap.add_argument("--row-order", action="store_true", help="GGUF row order (the slab kernel) instead of the tiled order")
    ap.add_argument("--reps", type=int, default=20)
    args = ap.parse_args()
    if args.build:
        return build()
    import numpy as np
    import torch

    import qwen_llm_amd as dfl

    L = C.CDLL(TRACE_LIB)
    vp, i32, i64, sz = C.c_void_p, C.c_int32, C.c_int64, C.c_size_t
    L.dflash_ctx_create.argtypes = [i32, sz, C.POINTER(vp)]
    L.dflash_gemm_fewrow.argtypes = [vp, i32, vp, vp, i32, vp, i64, i64, i32, vp]
    L.dflash_repack_q4k_tiled.argtypes = [vp, vp, vp, i64, i64, vp]
    L.dflash_q4k_tiled_bytes.argtypes = [i64, i64]
    L.dflash_q4k_tiled_bytes.restype = sz
    L.dflash_dbg_set_trace.argtypes = [C.c_uint64]
    L.dflash_dbg_set_trace2.argtypes = [C.c_uint64]
    ctx = vp()
    assert L.dflash_ctx_create(0, 0, C.byref(ctx)) == 0
    n_in, n_out, n_wg, n_sets = args.n_in, args.n_out, 256, 8
    g = torch.Generator(device="cuda")
    g.manual_seed(1)
    ws = []
    for _ in range(n_sets):
        w = dfl.synth.random_blocks_device(dfl.synth.Q4_K, n_out, n_in, 0.02, g, "cuda")
        if not args.row_order:
            t = torch.empty(L.dflash_q4k_tiled_bytes(n_in, n_out), dtype=torch.uint8, device="cuda")
            assert L.dflash_repack_q4k_tiled(ctx, w.data_ptr(), t.data_ptr(), n_in, n_out, None) == 0
            torch.cuda.synchronize()
            w = t
        ws.append(w)
    wt = dfl.TYPE_Q4_K if args.row_order else dfl.TYPE_Q4_K_TILED
    x = torch.randn((16, n_in), device="cuda", generator=g).half()
    y = torch.empty((16, n_out), device="cuda")

    def run(k):
        assert L.dflash_gemm_fewrow(ctx, wt, ws[k % n_sets].data_ptr(), x.data_ptr(), dfl.TYPE_F16, y.data_ptr(), n_in, n_out, 16, None) == 0

    for k in range(16):
        run(k)
    torch.cuda.synchronize()
    tr = torch.zeros(n_wg * 16, dtype=torch.int64, device="cuda")
    tr2 = torch.zeros(n_wg * 16 * 8, dtype=torch.int64, device="cuda")
    L.dflash_dbg_set_trace(tr.data_ptr())
    L.dflash_dbg_set_trace2(tr2.data_ptr())
    first, last = [[] for _ in NAMES], [[] for _ in NAMES]
    for rep in range(args.reps):
        run(rep)
        run(rep + 1)  # back to back, as in a model
        torch.cuda.synchronize()
        h = tr.cpu().numpy().reshape(n_wg, 16)
        h2 = tr2.cpu().numpy().reshape(n_wg, 16, 8)
        t0 = h[:, 0][h[:, 0] > 0].min()
        for wg in range(n_wg):
            if h[wg, 0] == 0:
                continue
            for i in range(len(NAMES)):
                v = h2[wg, :, i]
                v = v[v > 0]
                if v.size:
                    first[i].append((v.min() - t0) * 0.01)
                    last[i].append((v.max() - t0) * 0.01)
    print(f"{'Q4_K row order (slab kernel)' if args.row_order else 'Q4_K tiled order'}, {n_in} -> {n_out}, 16 rows f16; microseconds after the "
          f"earliest workgroup's start, over {args.reps} launches x {n_wg} workgroups (first / last wave of a workgroup)")
    for i in (0, 1, 2, 4, 5, 6, 7, 3):
        if first[i]:
            a, b = np.array(first[i]), np.array(last[i])
            print(f"  {NAMES[i]:26s} first wave: mean {a.mean():6.2f}  p10 {np.percentile(a, 10):6.2f}  p90 {np.percentile(a, 90):6.2f}   "
                  f"last wave: mean {b.mean():6.2f}  p10 {np.percentile(b, 10):6.2f}  p90 {np.percentile(b, 90):6.2f}")


if __name__ == "__main__":
    main()
