"""There is no fallback: without a GPU, without a compiler or with a source that does not build,
the framework says so and stops."""
import os
import subprocess
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(torch.cuda.is_available(), reason="needs a machine without a GPU")
def test_engine_refuses_to_run_without_a_gpu():
    from agave_amd.engine import Engine
    import plain_gemma3 as P
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        Engine.from_random(P.tiny_config("A"), seed=0, dtype="float32")


def test_missing_compiler_is_an_error_not_a_fallback(tmp_path):
    """With no hipcc to be found and nothing built, loading a kernel library raises."""
    code = (
        "import os, sys\n"
        f"sys.path.insert(0, {ROOT!r})\n"
        "from agave_amd.ops import library\n"
        "library.shutil.which = lambda name: None\n"
        "library.os.path.isfile = (lambda orig: (lambda p: False if str(p).endswith('hipcc') else orig(p)))(os.path.isfile)\n"
        "try:\n"
        "    library.load('elementwise')\n"
        "except library.KernelLibraryError as e:\n"
        "    print('refused:', e)\n"
    )
    env = dict(os.environ, AGAVE_AMD_BUILD_DIR=str(tmp_path / "empty_build"), HIPCC="")
    # the in-tree build folder may hold a current object; point the search at an empty folder only
    code = code.replace("from agave_amd.ops import library\n",
                        "from agave_amd.ops import library\n"
                        "library._find_built = lambda name, digest: None\n")
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env, timeout=120)
    assert "refused:" in out.stdout and "hipcc not found" in out.stdout, out.stdout + out.stderr


def test_a_source_that_does_not_build_is_reported_with_the_compiler_output(tmp_path):
    from agave_amd.ops import library
    bad = tmp_path / "csrc"
    bad.mkdir()
    (bad / "broken.hip").write_text("this is not C++\n")
    old_csrc, old_env = library.CSRC, os.environ.get("AGAVE_AMD_BUILD_DIR")
    library.CSRC = str(bad)
    os.environ["AGAVE_AMD_BUILD_DIR"] = str(tmp_path / "build")
    try:
        with pytest.raises(library.KernelLibraryError, match="hipcc failed for broken"):
            library._compile_many(["broken"])
    finally:
        library.CSRC = old_csrc
        if old_env is None:
            os.environ.pop("AGAVE_AMD_BUILD_DIR", None)
        else:
            os.environ["AGAVE_AMD_BUILD_DIR"] = old_env
