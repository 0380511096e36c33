"""include/amct_hip.h must be valid C (the boundary a cgo / JNI / ctypes binding compiles against)."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_header_compiles_as_c99_and_as_cpp(tmp_path):
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no C compiler")
    src = tmp_path / "use_header.c"
    src.write_text('#include "amct_hip.h"\n'
                   'int probe(void) { return amct_hip_version() + AMCT_E_TOO_LARGE + AMCT_COL_MINMAX_NOALLOC_MAX_COLS\n'
                   '                  + (int)sizeof(amct_stream_t) + AMCT_BF16 + AMCT_STAGE_COL + AMCT_CODES_I32; }\n')
    inc = os.path.join(ROOT, "include")
    for std, lang in (("-std=c99", "c"), ("-std=c11", "c"), ("-std=c++11", "c++")):
        p = subprocess.run([gcc, "-x", lang, std, "-pedantic", "-Wall", "-Werror", "-I", inc, "-c", str(src), "-o",
                            str(tmp_path / "o.o")], capture_output=True, text=True)
        assert p.returncode == 0, p.stderr
