"""The geometry that the NCDHW-direct convolution kernel, its planner and its launch share
(amos_amd/csrc/conv_nchw_geom.h), played on the CPU: tests/conv_nchw_geom_check.cpp writes every
tile's patch into a model of LDS with the kernel's writer addresses and asks the readers' address
function for every (output position, tap, chunk): the element the convolution wants or zero
padding, no slot written twice, nothing outside the buffer, no LDS bank slot used by more than two
lanes of a half wave in a fragment read, the weight tile's slot <-> (row, chunk) maps inverse to
each other."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_conv_nchw_geometry_on_the_cpu(tmp_path):
    exe = str(tmp_path / "geom_check")
    subprocess.check_call(["g++", "-O1", "-I", os.path.join(ROOT, "amos_amd", "csrc"), "-o", exe,
                           os.path.join(ROOT, "tests", "conv_nchw_geom_check.cpp")])
    out = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=300)
    text = out.stdout.decode()
    assert out.returncode == 0 and text.strip().endswith("ok"), text[-2000:]
