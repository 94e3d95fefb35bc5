"""Build libarhip.so (HIP kernels + C ABI) for gfx950 with hipcc.

    python -m autorust_amd.build          # rebuild if sources are newer
    python -m autorust_amd.build --force

hipcc cross-compiles without a GPU.  The library lands in-tree
(autorust_amd/libarhip.so) so that it travels with the source tree.
"""
import os
import struct
import subprocess
import sys
import time

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libarhip.so")
PROBES = os.path.join(HERE, "probes.hsaco")
KERNELS = os.path.join(HERE, "attn_kernels.hsaco")  # the named entry points (csrc/attn_entry.hip)
HOST_LIB = os.path.join(HERE, "libautorust_host.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# the pipelined kernel's variants compile in translation units of their own (pipe_launch.h), side by side
SOURCES = ["device.hip", "flash.hip", "sage_quant.hip", "pipe_bf16.hip", "pipe_i8.hip", "pipe_i8_keys.hip", "pipe_i8_qf.hip",
           "pipe_i8_keys_qf.hip", "pipe_fp8.hip", "pipe_fp8_qf.hip", "pipe_fp8_keys.hip"]
HEADERS = ["arhip_internal.h", "attn_fwd.h", "attn_pipe.h", "pipe_launch.h", "pipe_tu.h", "flash_f32.h", "flash_bwd_f32.h",
           "sage_quant_kernels.h", os.path.join("..", "..", "include", "arhip.h")]
ENTRY_PARTS = 15  # code objects csrc/attn_entry.hip compiles as (-DARHIP_ENTRY_PART=k), packed into KERNELS

# -packed-fp32-ops off: packed fp32 VALU instructions are not used by this build.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wall", "-Wno-unused-function", "-Wno-inline-asm",
         # loop strength reduction multiplies the address registers of the tile loop and spills them
         "-mllvm", "-disable-lsr"]


def _newer(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + r.stdout + r.stderr)
        raise RuntimeError("hipcc failed")
    # the host pass does not know the packed-fp32 feature and says so; that is harmless
    noise = "is not a recognized feature for this target"
    out = "\n".join(l for l in (r.stdout + r.stderr).splitlines() if noise not in l)
    if out.strip():
        sys.stderr.write(out + "\n")


def build(force=False, verbose=False):
    noise = "is not a recognized feature for this target"
    srcs = [os.path.join(CSRC, s) for s in SOURCES]
    headers = [os.path.join(CSRC, h) for h in HEADERS]
    deps = srcs + headers + [os.path.abspath(__file__)]
    entry_src = os.path.join(CSRC, "attn_entry.hip")
    probe_src = os.path.join(CSRC, "probes.hip")
    # every hipcc job that is due is queued (the objects of libarhip.so, the parts of the entry-point code object, the
    # probes) and MAX_JOBS of them run at a time, in the order queued
    objs, jobs = [], []
    build_lib = force or _newer(LIB, deps)

    def start(cmd):
        jobs.append(cmd)

    if build_lib:
        for s in srcs:
            o = s[:-4] + ".o"
            objs.append(o)
            start([HIPCC] + FLAGS + ["-c", s, "-o", o])
    parts = []
    if force or _newer(KERNELS, [entry_src] + headers):
        for k in range(1, ENTRY_PARTS + 1):
            parts.append(os.path.join(CSRC, "attn_entry.part%d.co" % k))
            start([HIPCC] + FLAGS + ["-DARHIP_ENTRY_PART=%d" % k, "--genco", entry_src, "-o", parts[-1]])
    if os.path.exists(probe_src) and (force or _newer(PROBES, [probe_src])):
        start([HIPCC] + FLAGS + ["--genco", probe_src, "-o", PROBES])
    failed = False
    limit = max(1, min(int(os.environ.get("MAX_JOBS", os.cpu_count() or 4)), 16))
    running, queue = [], list(jobs)
    while queue or running:
        while queue and len(running) < limit:
            cmd = queue.pop(0)
            if verbose:
                print(" ".join(cmd), flush=True)
            log = open(cmd[-1] + ".log", "w+")   # beside the job's output file; removed below
            running.append((cmd, subprocess.Popen(cmd, stdout=log, stderr=subprocess.STDOUT, text=True), log))
        time.sleep(0.2)
        for item in list(running):
            cmd, p, log = item
            if p.poll() is None:
                continue
            running.remove(item)
            log.seek(0)
            # the host pass does not know the packed-fp32 feature and says so; that is harmless
            out = "\n".join(l for l in log.read().splitlines() if noise not in l)
            log.close()
            os.remove(cmd[-1] + ".log")
            if p.returncode != 0:
                sys.stderr.write(" ".join(cmd) + "\n" + out + "\n")
                failed = True
            elif out.strip():
                sys.stderr.write(out + "\n")
    if failed:
        raise RuntimeError("hipcc failed")
    if parts:
        # one file for the seam: "ARHIPKO1", count, then every part with its size, padded to 16 bytes (arhip_module_load)
        blob = b"ARHIPKO1" + struct.pack("<II", len(parts), 0)
        for part in parts:
            data = open(part, "rb").read()
            blob += struct.pack("<Q", len(data)) + data + b"\0" * (-len(data) % 16)
            os.remove(part)
        with open(KERNELS, "wb") as f:
            f.write(blob)
    if build_lib:
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
    # C++ mirror of the reference's attention interface (+ the flat C shim the tests drive it with)
    host_srcs = [os.path.join(CSRC, "host", f) for f in ("autorust_host.cpp", "host_capi.cpp")]
    host_deps = host_srcs + [os.path.join(CSRC, "host", "autorust_host.h"), LIB]
    if force or _newer(HOST_LIB, host_deps):
        _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-o", HOST_LIB] + host_srcs +
             ["-L" + HERE, "-larhip", "-Wl,-rpath,$ORIGIN"])
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv, verbose=True)
    print(LIB)
