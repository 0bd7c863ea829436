"""The boundary as a compiler sees it: include/rof.h and include/rof_bench.h are valid C11 and C++17 on their own,
the struct sizes that the ctypes binding assumes are the compiler's, and the C++ operator module that binds the C
ABI (artifact_amd/csrc/rof_torch.cpp, the text that the integration guide shows) is built and loads.  No GPU."""
import os
import shutil
import subprocess
import sys
import textwrap

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INC = os.path.join(ROOT, "include")


@pytest.mark.parametrize("compiler,std,suffix", [("gcc", "-std=c11", ".c"), ("g++", "-std=c++17", ".cpp")])
def test_headers_compile_on_their_own_and_agree_with_the_ctypes_structs(tmp_path, compiler, std, suffix):
    if not shutil.which(compiler):
        pytest.skip(compiler + " not installed")
    body = textwrap.dedent("""
        #include "rof_bench.h"   /* includes rof.h */
        #include <stdio.h>
        int main(void) {
            /* every entry point is referenced, so a declaration that does not parse or a type that is missing fails here */
            void *fns[] = {(void *)rof_strerror, (void *)rof_plan_build, (void *)rof_layout_from_v2, (void *)rof_layout_from_v1,
                           (void *)rof_layout_from_parts, (void *)rof_layout_upload, (void *)rof_layout_set_degrees,
                           (void *)rof_aggregate, (void *)rof_aggregate_epilogue, (void *)rof_aggregate_noalloc,
                           (void *)rof_column_sums, (void *)rof_layout_stats_n, (void *)rof_layout_set_tuning,
                           (void *)rof_aggregate_timed, (void *)rof_device_read};
            printf("%d %d %d %d %d\\n", (int)sizeof(rof_layout_opts), (int)sizeof(rof_epilogue), (int)sizeof(rof_launch_tuning),
                   ROF_ABI_VERSION, (int)(sizeof(fns) / sizeof(fns[0])));
            return 0;
        }
        """)
    # the probe only takes addresses, so it links against the built library
    src = tmp_path / ("probe" + suffix)
    src.write_text(body)
    exe = tmp_path / "probe"
    lib_dir = os.path.join(ROOT, "artifact_amd")
    subprocess.run([compiler, std, "-Wall", "-Werror", "-I", INC, str(src), "-o", str(exe), "-L", lib_dir, "-l:librof.so",
                    "-Wl,-rpath," + lib_dir, "-Wl,--allow-shlib-undefined"], check=True)
    # (not run: loading librof.so would pull in the HIP runtime; the sizes are compile-time constants, read back below)
    probe = tmp_path / ("sizes" + suffix)
    probe.write_text('#include "rof_bench.h"\n#include <stdio.h>\nint main(void) { printf("%d %d %d %d\\n", '
                     "(int)sizeof(rof_layout_opts), (int)sizeof(rof_epilogue), (int)sizeof(rof_launch_tuning), "
                     "ROF_ABI_VERSION); return 0; }\n")
    exe2 = tmp_path / "sizes"
    subprocess.run([compiler, std, "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", INC, str(probe), "-o", str(exe2)], check=True)
    out = subprocess.run([str(exe2)], check=True, capture_output=True, text=True).stdout.split()
    import ctypes as C

    from artifact_amd import _lib

    assert [int(v) for v in out[:3]] == [C.sizeof(_lib.LayoutOpts), C.sizeof(_lib.Epilogue), C.sizeof(_lib.LaunchTuning)]
    assert int(out[3]) == _lib.lib().rof_version()


def test_compiled_operator_module_is_built_and_exports_the_upstream_functions():
    """artifact_amd/_ROF*.so is csrc/rof_torch.cpp compiled against PyTorch's headers and include/rof.h (by
    artifact_amd/build.py): the C++ binding of the C ABI has met a compiler and links.  The calls fail before any
    GPU work with upstream's CHECK_INPUT message (reuse_conv.cpp:121-123)."""
    import torch

    from artifact_amd import rof_module
    from artifact_amd.build import torch_module_path

    assert os.path.exists(torch_module_path()), "run `python -m artifact_amd.build`"
    mod = rof_module.compiled()
    for name in ("SAG", "GNNA_forward", "GNNA_backward", "reuse_forward_v1", "reuse_backward_v1", "reuse_forward_v2",
                 "reuse_backward_v2"):
        assert callable(getattr(mod, name))
    x = torch.zeros(3, 4)
    i = torch.zeros(3, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="input must be a CUDA tensor"):
        mod.GNNA_forward(x, x, i, x, i, i, 3, 32, 4)
    with pytest.raises(TypeError):                                      # upstream's positional signature, nothing more
        mod.reuse_forward_v2(x, x, i, x, i, i, i, 3, 32, 4, None)
    assert rof_module.install("ROF_compiled_for_test") is mod and sys.modules.pop("ROF_compiled_for_test") is mod


def test_integration_doc_shows_the_compiled_source():
    """The C++ binding that the integration guide shows is quoted from csrc/rof_torch.cpp, not written beside it."""
    doc = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    src = open(os.path.join(ROOT, "artifact_amd", "csrc", "rof_torch.cpp")).read()
    start = doc.index("```cpp", doc.index("### 3.2")) + len("```cpp\n")
    quoted = doc[start:doc.index("```", start)]
    blocks = [b for b in quoted.split("// ...\n") if b.strip()]
    assert blocks, "no quoted source"
    for b in blocks:
        assert b in src, "the integration guide quotes text that is not in csrc/rof_torch.cpp:\n" + b[:200]
