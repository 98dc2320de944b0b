"""Builds libcntk_amd_quantizer.so (HIP, gfx950) in-tree with hipcc. Run: python -m cntk_amd.build"""
import os
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libcntk_amd_quantizer.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # the CPU reference never fuses multiply-add; bit-exact codes and residuals need the same here
    "-ffp-contract=off",
    # no packed fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


# The library's source files share no device code and are compiled side by side: the C ABI (float matrices and everything
# independent of the element type), one file per kernel family of the float instantiation, and the double instantiation.
SOURCES = ["quantizer_api.hip", "quantizer_family_tile.hip", "quantizer_family_column.hip", "quantizer_family_register_256.hip",
           "quantizer_family_register_1024.hip", "quantizer_family_register_edge.hip", "quantizer_family_strip.hip",
           "quantizer_family_stripe_register_256.hip", "quantizer_family_stripe_register_1024.hip", "quantizer_family_unquantize.hip",
           "quantizer_family_batch_quantize.hip", "quantizer_family_batch_stripe.hip", "quantizer_api_f64.hip"]
# compilers running at once (a source file takes up to 3 GB while it is compiled)
JOBS = max(1, min(16, os.cpu_count() or 1, int(os.environ.get("MAX_JOBS", "16"))))


def resource_report_path(source):
    """Where build_library leaves the compiler's per-kernel resource figures of a source file: one line per kernel,
    `name=<mangled> VGPRs=.. ScratchSize=.. Occupancy=.. VGPRsSpill=.. SGPRsSpill=..` (scratch in bytes per lane)."""
    return os.path.join(HERE, "csrc", "build", os.path.splitext(source)[0] + ".resources.txt")


def split_resource_remarks(stderr):
    """Separates hipcc's kernel-resource-usage remarks from the rest of its output; returns ([{field: value} per kernel],
    [other lines])."""
    fields = {"TotalSGPRs": "SGPRs", "VGPRs": "VGPRs", "ScratchSize [bytes/lane]": "ScratchSize", "Occupancy [waves/SIMD]": "Occupancy",
              "SGPRs Spill": "SGPRsSpill", "VGPRs Spill": "VGPRsSpill", "LDS Size [bytes/block]": "LDS"}
    kernels, rest, skip = [], [], 0
    for line in stderr.splitlines():
        if "[-Rpass-analysis=kernel-resource-usage]" in line:
            body = line.split("remark:", 1)[1].rsplit("[-Rpass-analysis", 1)[0].strip()
            key, _, value = body.partition(":")
            if key.strip() == "Function Name":
                kernels.append({"name": value.strip()})
            elif kernels and key.strip() in fields:
                kernels[-1][fields[key.strip()]] = value.strip()
            skip = 2  # the source line and the caret that follow a remark
        elif skip > 0 and (line.lstrip().startswith("|") or line.lstrip()[:1].isdigit() or line.startswith("In file included")):
            skip -= 1
        elif line.startswith("In file included from"):
            continue
        else:
            rest.append(line)
    return kernels, rest


def build_library(verbose=False, only=None):
    """Compiles the sources (or, with `only`, just the named ones, keeping the other object files) and links the
    library."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    obj_dir = os.path.join(HERE, "csrc", "build")
    os.makedirs(obj_dir, exist_ok=True)
    objs = []
    todo = []
    for name in SOURCES:
        obj = os.path.join(obj_dir, os.path.splitext(name)[0] + ".o")
        objs.append(obj)
        if only is not None and name not in only and os.path.exists(obj):
            continue
        # the compiler reports every kernel's registers, scratch memory and occupancy: kept beside the object file
        todo.append((name, [hipcc] + HIPCC_FLAGS + ["-Rpass-analysis=kernel-resource-usage", "-c", "-o", obj, os.path.join(HERE, "csrc", name)]))
    errors = []
    running = []

    def reap(proc_entry):
        name, proc, log = proc_entry
        proc.wait()
        log.seek(0)
        stderr = log.read()
        log.close()
        remarks, rest = split_resource_remarks(stderr)
        # the host pass does not know the packed-fp32 feature and says so; that warning is harmless
        err = "\n".join(l for l in rest if "packed-fp32-ops" not in l)
        if proc.returncode != 0:
            errors.append("%s:\n%s" % (name, err))
            return
        with open(resource_report_path(name), "w") as f:
            for kernel in remarks:
                f.write(" ".join("%s=%s" % kv for kv in kernel.items()) + "\n")
        if verbose and err.strip():
            print(err, file=sys.stderr)

    for name, cmd in todo:
        while len(running) >= JOBS:
            reap(running.pop(0))
        if verbose:
            print(" ".join(cmd), flush=True)
        log = tempfile.TemporaryFile(mode="w+")  # (not a pipe: hundreds of remarks would fill it while the compiler waits its turn to be read)
        running.append((name, subprocess.Popen(cmd, stdout=subprocess.DEVNULL, stderr=log, text=True), log))
    for entry in running:
        reap(entry)
    if errors:
        raise RuntimeError("hipcc failed:\n" + "\n".join(errors))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("linking the library failed:\n" + res.stderr)
    return LIB_PATH


CPP_TESTS = ["test_matrix_quantizer", "test_allreduce_aggregator", "test_distributed_learner", "test_quantized_communicator", "test_v2_aggregator",
             "bench_allreduce"]


def build_cpp_tests(verbose=False):
    """Compiles the C++ programs under tests/cpp (host mirror classes, aggregator, all-reduce timing) against the
    library and the CPU oracle."""
    root = os.path.dirname(HERE)
    out_dir = os.path.join(root, "tests", "cpp", "bin")
    os.makedirs(out_dir, exist_ok=True)
    oracle_dir = os.path.join(root, "oracle")
    subprocess.run(["make", "-C", oracle_dir, "all"], check=True, capture_output=True)
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    exes = []
    for name in CPP_TESTS:
        src = os.path.join(root, "tests", "cpp", name + ".cpp")
        if not os.path.exists(src):
            continue
        exe = os.path.join(out_dir, name)
        # plain host C++ (no device code): the mirror classes only call the C ABI and the HIP runtime API
        cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-Wall", "-pthread", src,
               "-D__HIP_PLATFORM_AMD__", "-I" + os.path.join(rocm, "include"), "-o", exe,
               "-L" + HERE, "-lcntk_amd_quantizer", "-L" + oracle_dir, "-loracle",
               "-L" + os.path.join(rocm, "lib"), "-lamdhip64", "-Wl,-rpath," + os.path.join(rocm, "lib"),
               "-Wl,-rpath,$ORIGIN/../../../cntk_amd", "-Wl,-rpath,$ORIGIN/../../../oracle"]
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError("building %s failed:\n%s" % (name, res.stderr))
        exes.append(exe)
    return exes


if __name__ == "__main__":
    # python -m cntk_amd.build [source file names ...]: recompile only those (a development shortcut)
    print(build_library(verbose=True, only=sys.argv[1:] or None))
    print(build_cpp_tests(verbose=True))
