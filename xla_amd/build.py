"""Builds libxla_amd_qmm.so (gfx950) in-tree with hipcc.

`python -m xla_amd.build` compiles every .hip file of xla_amd/csrc and links
them into xla_amd/libxla_amd_qmm.so.  hipcc cross-compiles, so no GPU is
needed to build.
"""
import concurrent.futures
import os
import json
import re
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
OBJ_DIR = os.path.join(PKG_DIR, "csrc", "build")
LIB_PATH = os.path.join(PKG_DIR, "libxla_amd_qmm.so")

# (source, extra flags, object name); the skinny kernels are built once per
# activation dtype and the weight-only GEMM once per (dtype, row tile) so that
# the units compile in parallel
SOURCES = [
    # the slow units first: eight compilers run at a time
    ("qmm_wo_gemm.hip", ["-DQMM_WO_XT=1", "-DQMM_WO_MT=8"], "qmm_wo_gemm_bf16_mt8.o"),
    ("qmm_wo_gemm.hip", ["-DQMM_WO_XT=2", "-DQMM_WO_MT=8"], "qmm_wo_gemm_f16_mt8.o"),
    ("qmm_skinny.hip", ["-DQMM_SKINNY_XT=1"], "qmm_skinny_bf16.o"),
    ("qmm_skinny.hip", ["-DQMM_SKINNY_XT=2"], "qmm_skinny_f16.o"),
    ("qmm_skinny.hip", ["-DQMM_SKINNY_XT=0"], "qmm_skinny_f32.o"),
    ("qmm_skinny_resident.hip", ["-DQMM_SKINNY_XT=1"], "qmm_skinny_resident_bf16.o"),
    ("qmm_skinny_resident.hip", ["-DQMM_SKINNY_XT=2"], "qmm_skinny_resident_f16.o"),
    ("qmm_wo_gemm.hip", ["-DQMM_WO_XT=1", "-DQMM_WO_MT=4"], "qmm_wo_gemm_bf16_mt4.o"),
    ("qmm_wo_gemm.hip", ["-DQMM_WO_XT=2", "-DQMM_WO_MT=4"], "qmm_wo_gemm_f16_mt4.o"),
    ("qmm_wo_gemm_bw.hip", ["-DQMM_WO_BW_XT=1"], "qmm_wo_gemm_bw_bf16.o"),
    ("qmm_wo_gemm_bw.hip", ["-DQMM_WO_BW_XT=2"], "qmm_wo_gemm_bw_f16.o"),
    ("qmm_w8a8_gemm.hip", [], "qmm_w8a8_gemm.o"),
    ("qmm_api.hip", [], "qmm_api.o"),
    ("qmm_generic.hip", [], "qmm_generic.o"),
    ("qmm_quant_act.hip", [], "qmm_quant_act.o"),
    ("qmm_qdq.hip", [], "qmm_qdq.o"),
    ("qmm_linear.hip", [], "qmm_linear.o"),
]

# Diagnostic library: the same objects with the bf16 unit of the streaming kernel compiled with
# -DQMM_SKINNY_TIMELINE (every wave records when it reaches fixed points of the kernel; read back by
# `python bench.py --timeline`).  Never loaded by the operators.
TIMELINE_LIB_PATH = os.path.join(PKG_DIR, "libxla_amd_qmm_timeline.so")
TIMELINE_UNIT = ("qmm_skinny.hip", ["-DQMM_SKINNY_XT=1", "-DQMM_SKINNY_TIMELINE"], "qmm_skinny_bf16_timeline.o")
TIMELINE_REPLACES = "qmm_skinny_bf16.o"
DIAG_UNIT = ("qmm_diag.hip", [], "qmm_diag.o")  # diagnostic kernels: the diagnostic library only

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# packed-fp32 instructions are switched off on purpose (hipcc otherwise forms
# v_pk_*_f32 from scalar float code).
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-pass-failed",
    "-I", os.path.join(REPO_DIR, "include"), "-I", CSRC,
]


def _run(cmd):
  proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
  # The host pass does not know the device-only target feature; drop that line.
  out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
  if proc.returncode != 0:
    raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
  return out


# Every kernel of the library must keep its registers: a kernel that spills to scratch memory
# runs several times slower without failing any test.  The compiler reports each kernel's
# resources (-Rpass-analysis=kernel-resource-usage); the build reads the report, writes it to
# RESOURCES_PATH and refuses a kernel with a scratch frame.
RESOURCES_PATH = os.path.join(OBJ_DIR, "kernel_resources.json")
_REMARK = re.compile(r"remark:\s+(Function Name|VGPRs|AGPRs|ScratchSize \[bytes/lane\]|Occupancy \[waves/SIMD\]|"
                     r"LDS Size \[bytes/block\]): (\S+)")


def _kernel_resources(report: str, unit: str):
  kernels, cur = [], None
  for line in report.splitlines():
    m = _REMARK.search(line)
    if not m:
      continue
    key, val = m.group(1), m.group(2)
    if key == "Function Name":
      cur = {"unit": unit, "kernel": val}
      kernels.append(cur)
    elif cur is not None:
      cur[{"VGPRs": "vgprs", "AGPRs": "agprs", "ScratchSize [bytes/lane]": "scratch_bytes_per_lane",
           "Occupancy [waves/SIMD]": "waves_per_simd", "LDS Size [bytes/block]": "static_lds_bytes"}[key]] = int(val)
  return kernels


# Code bytes per kernel, read from the symbol table of the device code object inside each object file of this
# build.  A launch starts with a cold instruction cache, and the decode kernels run their straight-line prologue
# once: every instruction on the way to the first load is a few nanoseconds of a launch that lasts about twelve
# microseconds, so the two headline kernels have a budget, and the build fails when one of them outgrows it.
LLVM_BIN = os.environ.get("LLVM_BIN", "/opt/rocm/llvm/bin")
CODE_BUDGET_BYTES = {
    # mangled name of the kernel: bytes (decode GEMV, bf16 / int8 per channel, 16 rows at most; its persistent form)
    "_ZN12_GLOBAL__N_117qmm_skinny_kernelILi1ELi8ELi1ELi1ELi1ELb0ELb1ELi4ELi512EEEv10SkinnyArgs": 8192,
    "_ZN12_GLOBAL__N_126qmm_skinny_resident_kernelILi1ELb0EEEv10SkinnyArgs": 11264,
}


def _code_bytes(obj: str):
  """{kernel symbol: bytes} of the gfx950 code object bundled in `obj`."""
  fat, dev = obj + ".fatbin", obj + ".gfx950.co"
  try:
    _run(["objcopy", "-O", "binary", "--only-section=.hip_fatbin", obj, fat])
    _run([os.path.join(LLVM_BIN, "clang-offload-bundler"), "--type=o", "--targets=hipv4-amdgcn-amd-amdhsa--gfx950",
          "--input=" + fat, "--output=" + dev, "--unbundle"])
    table = _run([os.path.join(LLVM_BIN, "llvm-readelf"), "-sW", dev])
  finally:
    for f in (fat, dev):
      if os.path.exists(f):
        os.remove(f)
  sizes = {}
  for line in table.splitlines():
    f = line.split()
    if len(f) >= 8 and f[3] == "FUNC" and f[6] != "UND":
      sizes[f[7]] = int(f[2])
  return sizes


def build(verbose: bool = False, jobs: int = 8) -> str:
  os.makedirs(OBJ_DIR, exist_ok=True)
  objs = []

  def compile_one(item):
    src, extra, name = item
    obj = os.path.join(OBJ_DIR, name)
    out = _run([HIPCC] + FLAGS + ["-Rpass-analysis=kernel-resource-usage"] + extra +
               ["-c", os.path.join(CSRC, src), "-o", obj])
    kernels = _kernel_resources(out, name)
    sizes = _code_bytes(obj) if kernels else {}  # (a unit without kernels carries no device code object)
    for k in kernels:
      if k["kernel"] in sizes:
        k["code_bytes"] = sizes[k["kernel"]]
    if verbose:
      # (a remark is followed by the source line it points at and a caret line)
      rest = "\n".join(l for l in out.splitlines() if "kernel-resource-usage" not in l and
                       not re.match(r"^\s*\d*\s*\|", l) and l.strip() != "^")
      if rest.strip():
        print(rest)
    return obj, kernels

  with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
    results = list(ex.map(compile_one, SOURCES + [TIMELINE_UNIT, DIAG_UNIT]))
  diag_obj, diag_kernels = results.pop()
  timeline_obj, timeline_kernels = results.pop()
  objs = [r[0] for r in results]
  kernels = [k for r in results for k in r[1]]
  with open(RESOURCES_PATH, "w") as f:
    json.dump(kernels, f, indent=1)
  spilling = [k for k in kernels + timeline_kernels + diag_kernels if k.get("scratch_bytes_per_lane", 0) > 0]
  if spilling:
    raise RuntimeError("kernels with a scratch frame (register spills):\n" +
                       "\n".join("  %s: %s (%d bytes per lane, %d VGPRs)" % (k["unit"], k["kernel"], k["scratch_bytes_per_lane"],
                                                                            k.get("vgprs", -1)) for k in spilling))
  by_name = {k["kernel"]: k for k in kernels}
  over = []
  for name, budget in CODE_BUDGET_BYTES.items():
    k = by_name.get(name)
    if k is None or "code_bytes" not in k:
      raise RuntimeError("kernel with a code budget is not in the build (renamed?): " + name)
    if k["code_bytes"] > budget:
      over.append("  %s: %d bytes of code, budget %d" % (name, k["code_bytes"], budget))
  if over:
    raise RuntimeError("kernels over their code budget:\n" + "\n".join(over))
  tmp = LIB_PATH + ".tmp"
  _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", tmp] + objs)
  os.replace(tmp, LIB_PATH)
  tmp = TIMELINE_LIB_PATH + ".tmp"
  _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", "-o", tmp] +
       [timeline_obj if os.path.basename(o) == TIMELINE_REPLACES else o for o in objs] + [diag_obj])
  os.replace(tmp, TIMELINE_LIB_PATH)
  return LIB_PATH


if __name__ == "__main__":
  path = build(verbose=True)
  print("built", path)
  sys.exit(0)
