"""Build the native libraries of this package in-tree.

`python -m oxillama_amd.build` compiles
  * oxillama_amd/liboxq_hip.so   -- HIP kernels + C ABI (include/oxq.h), gfx950 only
  * oxillama_amd/liboxq_synth.so -- host-side synthetic weight generator
  * oxillama_amd/liboxq_benchkit.so -- copy / streaming-read kernels for measurement calibration
  * tests/cpp/test_quant_kernel.bin -- C++ mirror of the reference interface + its replayed unit tests
hipcc cross-compiles gfx950 code objects without a GPU present.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
HIP_SOURCES = ["oxq_api.hip", "oxq_gemv.hip", "oxq_gemv_more.hip", "oxq_gemv_f32.hip", "oxq_gemm.hip", "oxq_gemm_more.hip", "oxq_gemm_prefill.hip", "oxq_quantize.hip", "oxq_linear.hip", "oxq_gguf.hip", "oxq_topk.hip", "oxq_lm_head.hip", "oxq_moe.hip"]
HIP_LIB = os.path.join(HERE, "liboxq_hip.so")
SYNTH_LIB = os.path.join(HERE, "liboxq_synth.so")
BENCHKIT_LIB = os.path.join(HERE, "liboxq_benchkit.so")
CPP_TEST_BIN = os.path.join(os.path.dirname(HERE), "tests", "cpp", "test_quant_kernel.bin")

# -ffp-contract=off: the fp32 epilogues follow the reference's operation order (Rust
# never fuses a*b+c).  Packed fp32 instructions are switched off.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)


def build_hip(extra=()):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    from concurrent.futures import ThreadPoolExecutor
    objs = [os.path.join(CSRC, src.replace(".hip", ".o")) for src in HIP_SOURCES]
    with ThreadPoolExecutor(max_workers=min(len(HIP_SOURCES), 6)) as pool:  # one hipcc per translation unit
        list(pool.map(lambda so: run([hipcc, *HIPCC_FLAGS, *extra, "-c", os.path.join(CSRC, so[0]), "-o", so[1]]),
                      zip(HIP_SOURCES, objs)))
    run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", HIP_LIB, *objs])
    return HIP_LIB


def build_synth():
    run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-pthread", "-ffp-contract=off",
         "-o", SYNTH_LIB, os.path.join(CSRC, "synth.cpp")])
    return SYNTH_LIB


def build_benchkit():
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    run([hipcc, *HIPCC_FLAGS, "-shared", "-o", BENCHKIT_LIB, os.path.join(CSRC, "benchkit.hip")])
    return BENCHKIT_LIB


def build_cpp_tests():
    """The C++ mirror of the reference interface (include/oxq/quant_kernel.hpp) and the
    program that replays the reference's unit tests through it."""
    root = os.path.dirname(HERE)
    run(["g++", "-O1", "-std=c++17", "-Wall", "-I", os.path.join(root, "include"),
         os.path.join(root, "tests", "cpp", "test_quant_kernel.cpp"), "-o", CPP_TEST_BIN,
         "-L", HERE, "-loxq_hip", "-Wl,-rpath,$ORIGIN/../../oxillama_amd",
         "-Wl,-rpath-link,/opt/rocm/lib", "-Wl,--allow-shlib-undefined"])
    return CPP_TEST_BIN


def build_all():
    build_hip()
    build_synth()
    build_benchkit()
    build_cpp_tests()


if __name__ == "__main__":
    build_all()
    sys.exit(0)
