"""TEST INFRASTRUCTURE ONLY (an address checker, not an execution path: values that cross threads are not reproduced).

Bounds check of generated kernels on the CPU: the generated translation unit of a module (its main.hip and the
device prelude it includes, unchanged) is compiled for the host with tests/cpu_shim/host_builtins.h pre-included and
run thread by thread with every buffer (parameters, live-outs, the temp arena and every constant of the module, which
the generated source declares as arrays of the code object) placed against inaccessible guard pages, once flush with the
page before it (catches reads in front of a buffer) and once flush with the page behind it (catches reads past its end).
The workgroup's LDS is a buffer of exactly the kernel's dynamic LDS size whose end sits against a guard page.  An out-of-range access ends the run
with the buffer, the offset and the thread that made it."""
import json
import os
import re
import subprocess
import tempfile

from mononn_amd import MonoNNModule

HERE = os.path.dirname(os.path.abspath(__file__))
CLANG = "/opt/rocm/lib/llvm/bin/clang++"

DRIVER = r"""
#include <csignal>
#include <cstdio>
#include <cstdlib>
#include <sys/mman.h>
#include <unistd.h>
Dim3 threadIdx, blockIdx, gridDim, blockDim;
char* mononn_lds;   // the kernel's `smem`: launch_dims()["smem"] bytes, the last of them in front of a guard page
%(const_decls)s
#include "main.hip"

struct Buf { const char* name; size_t bytes; char* base; char* lo; char* hi; };
static Buf bufs[%(nbuf)d];
static const size_t kGuard = size_t(64) << 20;
static void on_fault(int, siginfo_t* si, void*) {
  char* a = static_cast<char*>(si->si_addr);
  for (auto& b : bufs)
    if (a >= b.lo && a < b.hi) {
      std::fprintf(stderr, "OUT OF BOUNDS: %%s (%%zu bytes) at byte offset %%ld, block %%u thread %%u\n", b.name, b.bytes, long(a - b.base), blockIdx.x, threadIdx.x);
      _exit(3);
    }
  std::fprintf(stderr, "FAULT at %%p outside every buffer's guard range, block %%u thread %%u\n", (void*)a, blockIdx.x, threadIdx.x);
  _exit(4);
}
int main(int argc, char** argv) {
  const bool at_end = argc > 1 && argv[1][0] == 'e';
  const char* names[] = {%(names)s};
  const size_t sizes[] = {%(sizes)s};
  const long page = sysconf(_SC_PAGESIZE);
  for (int i = 0; i < %(nbuf)d; ++i) {
    const size_t body = (std::max<size_t>(sizes[i], 1) + page - 1) / page * page;
    char* r = static_cast<char*>(mmap(nullptr, body + 2 * kGuard, PROT_NONE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0));
    if (r == MAP_FAILED) { std::perror("mmap"); return 2; }
    mprotect(r + kGuard, body, PROT_READ | PROT_WRITE);
    char* base = at_end ? r + kGuard + ((body - sizes[i]) & ~size_t(15)) : r + kGuard;
    for (size_t k = 0; k < sizes[i]; ++k) base[k] = char(k * 7 + i);     // finite halves, small integers as indices
    bufs[i] = {names[i], sizes[i], base, r, r + body + 2 * kGuard};
  }
%(const_binds)s
  mononn_lds = bufs[%(lds_index)d].lo + kGuard + ((((std::max<size_t>(sizes[%(lds_index)d], 1) + page - 1) / page * page) - sizes[%(lds_index)d]) & ~size_t(15));
  bufs[%(lds_index)d].base = mononn_lds;
  struct sigaction sa = {};
  sa.sa_sigaction = on_fault;
  sa.sa_flags = SA_SIGINFO;
  sigaction(SIGSEGV, &sa, nullptr);
  sigaction(SIGBUS, &sa, nullptr);
  gridDim.x = %(grid)d;
  blockDim.x = %(block)d;
  for (unsigned b = 0; b < %(grid)du; ++b)
    for (unsigned t = 0; t < %(block)du; ++t) {
      blockIdx.x = b;
      threadIdx.x = t;
      %(kernel)s(%(args)s);
    }
  std::printf("ok\n");
  return 0;
}
"""


def check_module(hlo_text, spec_json=None, workdir=None, opt="-O0", shrink=None):
    """Returns (ok, message).  -O0 keeps every load the generator wrote (an optimising build drops loads whose value
    goes unused, which is exactly what a misplaced load looks like); large kernels may need -O1 to finish in time.
    `shrink` = (buffer name, bytes) declares one buffer smaller than it is: the harness's own test, which must fail."""
    m = MonoNNModule.compile(hlo_text, spec_json, build=False)
    src = m.get_source("main.hip")
    info, dims = m.buffer_info(), m.launch_dims()
    names, sizes = [], []
    for i, b in enumerate(info["parameters"]):
        names.append(f"parameter {i}")
        sizes.append(b)
    for i, b in enumerate(info["liveouts"]):
        names.append(f"live-out {i}")
        sizes.append(b)
    names.append("temp arena")
    sizes.append(max(info["temp"], 16))
    # constants: `__device__ ... unsigned char buffer_for_<name>[bytes];` becomes a pointer into a guarded mapping
    consts = re.findall(r"^__device__ __attribute__\(\(aligned\(256\)\)\) unsigned char (buffer_for_\w+)\[(\d+)\];$", src, flags=re.M)
    src = re.sub(r"^__device__ __attribute__\(\(aligned\(256\)\)\) unsigned char (buffer_for_\w+)\[(\d+)\];$", r"// \1: \2 bytes, guarded by the driver", src, flags=re.M)
    n_args = len(names)
    for cname, cbytes in consts:
        names.append(cname)
        sizes.append(int(cbytes))
    names.append("LDS")
    sizes.append(max(dims["smem"], 16))
    lds_decl = "extern __shared__ __attribute__((aligned(16))) char smem[];"
    assert lds_decl in src, "the kernel's LDS declaration has changed"
    src = src.replace(lds_decl, "char* const smem = mononn_lds;")
    if shrink:
        sizes[names.index(shrink[0])] -= shrink[1]
    const_decls = "\n".join(f"unsigned char* {cname};" for cname, _ in consts)
    const_binds = "\n".join(f"  {cname} = reinterpret_cast<unsigned char*>(bufs[{n_args + i}].base);" for i, (cname, _) in enumerate(consts))
    tmp = workdir or tempfile.mkdtemp(prefix="mononn_cpu_bounds_")
    open(os.path.join(tmp, "main.hip"), "w").write(src)
    open(os.path.join(tmp, "headers.h"), "w").write(m.get_source("headers.h"))
    drv = DRIVER % {"nbuf": len(names), "names": ", ".join(json.dumps(n) for n in names), "sizes": ", ".join(f"{s}ul" for s in sizes),
                    "grid": dims["grid"], "block": dims["block"], "kernel": m.kernel_name,
                    "args": ", ".join(f"bufs[{i}].base" for i in range(n_args)), "const_decls": const_decls, "const_binds": const_binds, "lds_index": len(names) - 1}
    open(os.path.join(tmp, "driver.cpp"), "w").write(drv)
    exe = os.path.join(tmp, "driver")
    cp = subprocess.run([CLANG, "-x", "c++", "-std=c++17", opt, "-w", "-include", os.path.join(HERE, "cpu_shim", "host_builtins.h"), "-I", tmp,
                         os.path.join(tmp, "driver.cpp"), "-o", exe], capture_output=True, text=True)
    m.close()
    if cp.returncode != 0:
        return False, "host build failed:\n" + cp.stderr[-3000:]
    for mode in ("start", "end"):
        r = subprocess.run([exe, mode], capture_output=True, text=True, timeout=900)
        if r.returncode != 0:
            return False, f"buffers flush with their {mode}: " + (r.stderr.strip() or f"exit code {r.returncode}")
    return True, "ok"
