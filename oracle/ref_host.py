"""Builds the reference's own host translation unit — its task scheduler and Python module, hp_cuda.cpp — over this
library's drivers.  TEST INFRASTRUCTURE ONLY (used by tests/ and built by __graft_entry__.build()).

What it does is what a maintainer of the reference does to switch kernel layers: the block of nine hand-written
driver declarations (hp_cuda.cpp:18-102) becomes `#include "hp_cuda_shim.h"` + `#include "hp_cuda_shim_torch.h"`,
`hp_cuda_kernel.cu` is dropped and `libhpx.so` is linked instead.  The file is read where it lies under
/root/reference, edited in a temporary directory, passed through the source renames PyTorch-ROCm's extension build
applies to every extension (torch.utils.hipify: cudaStream_t -> hipStream_t, c10::cuda -> the HIP stream wrappers;
it also renames the file to hp_hip.cpp) and compiled with the host compiler.  No header, library or tool of the
reference's build is replaced by a stand-in, and nothing of the reference's text is kept: only the built module
lands in `out_dir` (default oracle/_ref/, which git ignores).

The result is a Python module `hp_cuda` whose init / submit_task / getResults / end and whose scheduler loops
(hp_cuda.cpp:163-772) are the reference's own code, calling this library's nine drivers.  tests/ run it on the GPU
to show the drivers behave under the reference's stream usage as the reference's drivers did.
"""
import os
import shutil
import subprocess
import sys
import sysconfig
import tempfile

REF = "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
PKG = os.path.join(ROOT, "torch-hipress-extension_amd")
OUT_DIR = os.path.join(HERE, "_ref")

# Edits beyond the swap of the declaration block and the hipify renames that the torch-1.3-era source needs to
# compile against this image's torch: (old text, new text, reason).  Empty: it compiles as it is.
EXTRA_EDITS = []

CALL_SITES = (  # the reference's own calls of the drivers must survive every edit untouched
    "hp_cuda_terngrad(in_floats, in_float_sizes, out_uint8_ts, out_uint8_t_sizes, bitwidths, enable_randoms, compute_stream);",
    "hp_cuda_terngradr(out_floats, out_float_sizes, in_uint8_ts, in_uint8_t_sizes, is_add_tos, compute_stream);",
    "hp_cuda_tbqr(out_floats, out_float_sizes, in_uint8_ts, in_uint8_t_sizes, thresholds_decomp, is_add_tos, compute_stream);",
    "hp_cuda_tbq(to_compress_floats, to_compress_float_sizes, residual_floats, residual_float_sizes, out_uint8_ts, out_uint8_t_sizes, thresholds_comp, compute_stream);",
)


def available():
    return os.path.exists(os.path.join(REF, "hp_cuda.cpp")) and os.path.exists(os.path.join(REF, "hp_cuda.h"))


def module_path(out_dir=OUT_DIR):
    return os.path.join(out_dir, "hp_cuda" + sysconfig.get_config_var("EXT_SUFFIX"))


def swapped_source():
    """hp_cuda.cpp with its lines 18-102 (the nine declarations) replaced by the two includes."""
    lines = open(os.path.join(REF, "hp_cuda.cpp")).read().split("\n")
    block = "\n".join(lines[17:102])
    assert block.lstrip().startswith("void hp_cuda_terngrad(") and block.rstrip().endswith(");"), block[:80]
    assert block.count("void hp_cuda_") == 9, "lines 18-102 no longer hold exactly the nine declarations"
    return "\n".join(lines[:17] + ['#include "hp_cuda_shim.h"', '#include "hp_cuda_shim_torch.h"'] + lines[102:])


def build(out_dir=OUT_DIR, verbose=False):
    """Returns (path of the built module, list of the extra edits applied).  Raises on failure."""
    import torch
    from torch.utils.hipify import hipify_python
    assert available(), "the reference's sources are not on this machine"
    os.makedirs(out_dir, exist_ok=True)
    with tempfile.TemporaryDirectory(prefix="ref_host_") as tmp:
        src_dir, hip_dir = os.path.join(tmp, "in"), os.path.join(tmp, "out")
        os.makedirs(src_dir)
        with open(os.path.join(src_dir, "hp_cuda.cpp"), "w") as f:
            f.write(swapped_source())
        shutil.copy(os.path.join(REF, "hp_cuda.h"), os.path.join(src_dir, "hp_cuda.h"))
        files = [os.path.join(src_dir, f) for f in ("hp_cuda.cpp", "hp_cuda.h")]
        res = hipify_python.hipify(project_directory=src_dir, output_directory=hip_dir, includes=[src_dir + "/*"],
                                   extra_files=files, is_pytorch_extension=True, show_detailed=False)
        cpp = [v.hipified_path for k, v in res.items() if os.path.basename(k) == "hp_cuda.cpp" and v.hipified_path]
        assert cpp, res
        cpp = cpp[0]
        text = open(cpp).read()
        applied = []
        for old, new, why in EXTRA_EDITS:
            assert old in text, f"edit no longer applies: {why}"
            text = text.replace(old, new)
            applied.append(why)
        for call in CALL_SITES:
            assert call in text, call
        with open(cpp, "w") as f:
            f.write(text)
        tdir = os.path.dirname(torch.__file__)
        so = module_path(out_dir)
        cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-w",
               "-DTORCH_API_INCLUDE_EXTENSION_H", "-DTORCH_EXTENSION_NAME=hp_cuda",
               f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", "-D__HIP_PLATFORM_AMD__", "-DUSE_ROCM",
               "-I" + os.path.dirname(cpp), "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(PKG, "csrc"),
               "-I" + os.path.join(tdir, "include"), "-I" + os.path.join(tdir, "include/torch/csrc/api/include"),
               "-I" + sysconfig.get_paths()["include"], "-I/opt/rocm/include",
               cpp, "-o", so,
               "-L" + PKG, "-lhpx", "-L" + os.path.join(tdir, "lib"), "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip",
               "-ltorch_hip", "-ltorch_python", "-L/opt/rocm/lib", "-lamdhip64", "-Wl,--no-undefined",
               "-Wl,-rpath," + os.path.relpath(PKG, out_dir).join(["$ORIGIN/", ""]), "-Wl,-rpath," + PKG,
               "-Wl,-rpath," + os.path.join(tdir, "lib")]
        libdir = sysconfig.get_config_var("LIBDIR")
        if libdir:
            cmd += ["-L" + libdir, f"-lpython{sys.version_info.major}.{sys.version_info.minor}"]
        if verbose:
            print("+", " ".join(cmd), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode:
            raise RuntimeError("compiling the reference's hp_cuda.cpp against the driver headers failed "
                               f"(extra edits applied: {applied}):\n{r.stderr[-8000:]}")
    return so, applied


if __name__ == "__main__":
    path, edits = build(verbose=True)
    print("built", path, "extra edits:", edits)
