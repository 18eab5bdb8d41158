"""Compiles mesh-llm_amd/csrc/*.hip into libmeshstage.so for gfx950 (hipcc cross-compiles without a GPU)."""
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libmeshstage.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    # never let the compiler emit packed-FP32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # leading scalar kernel arguments arrive in SGPRs at wave start instead of through a scalar load (kernels whose
    # start-up chain matters list those arguments first)
    "-mllvm", "-amdgpu-kernarg-preload-count=14",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
]


def _compile(src):
    obj = os.path.join(OBJ, os.path.basename(src) + ".o")
    cmd = [HIPCC, *FLAGS, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, " ".join(cmd), r.stderr))
    warn = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    return obj, warn


def build(verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")) + glob.glob(os.path.join(CSRC, "*.cpp")))
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        results = list(ex.map(_compile, srcs))
    if verbose:
        for obj, warn in results:
            if warn:
                print(warn, file=sys.stderr)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *[o for o, _ in results]]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (" ".join(cmd), r.stderr))
    return LIB


RPC_SRC = os.path.join(CSRC, "rpc")
RPC_SERVER = os.path.join(HERE, "rpc-server")


def build_rpc_server():
    """Links mesh-llm_amd/rpc-server: the rpc-server-compatible front end over libmeshstage.so (host code only; its
    buffers are HBM through the HIP runtime)."""
    srcs = [os.path.join(RPC_SRC, f) for f in ("rpc_main.cpp", "rpc_server.cpp", "rpc_graph.cpp", "rpc_graph_runner.cpp", "rpc_buffers_hip.cpp")]
    cmd = [HIPCC, "-O2", "-std=c++17", "-Wall", "-pthread", *srcs, "-L" + HERE, "-lmeshstage", "-Wl,-rpath,$ORIGIN", "-o", RPC_SERVER]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("rpc-server build failed:\n%s\n%s" % (" ".join(cmd), r.stderr))
    return RPC_SERVER


def build_rpc_server_hostmem(out_path):
    """The same server with tests/rpc_hostmem/buffers_host.cpp in place of the HIP buffers (g++ only): what the protocol
    tests run on a machine without a GPU.  Test infrastructure, never shipped."""
    root = os.path.dirname(HERE)
    srcs = [os.path.join(RPC_SRC, "rpc_main.cpp"), os.path.join(RPC_SRC, "rpc_server.cpp"), os.path.join(RPC_SRC, "rpc_graph.cpp"),
            os.path.join(root, "tests", "rpc_hostmem", "buffers_host.cpp"), os.path.join(root, "tests", "rpc_hostmem", "runner_host.cpp")]
    cmd = [os.environ.get("CXX", "g++"), "-O1", "-std=c++17", "-Wall", "-pthread", "-I" + RPC_SRC, *srcs, "-L" + HERE, "-lmeshstage", "-L/opt/rocm/lib",
           "-Wl,-rpath," + HERE, "-Wl,-rpath,/opt/rocm/lib", "-o", out_path]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("host-memory rpc-server build failed:\n%s\n%s" % (" ".join(cmd), r.stderr))
    return out_path


PLUGIN = os.path.join(HERE, "mesh-stage-plugin")


def build_plugin(out_path=PLUGIN):
    """Links mesh-llm_amd/mesh-stage-plugin: the stage as a mesh-llm plugin process with an inference endpoint (host code
    over the C ABI of libmeshstage.so)."""
    src = os.path.join(CSRC, "plugin", "plugin_main.cpp")
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-Wall", "-pthread", src, "-L" + HERE, "-lmeshstage", "-L/opt/rocm/lib",
           "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + HERE, "-Wl,-rpath,/opt/rocm/lib", "-o", out_path]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("mesh-stage-plugin build failed:\n%s\n%s" % (" ".join(cmd), r.stderr))
    return out_path


if __name__ == "__main__":
    print(build(verbose=True))
    print(build_rpc_server())
    print(build_plugin())
