"""Compiles and runs the host enumeration of the fragment-to-register maps (plain g++, no GPU)."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_fragment_maps_are_bijective_and_match_mfma_operand_layout(tmp_path):
    exe = tmp_path / "fragment_map_check"
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-o", str(exe),
                           os.path.join(ROOT, "tests", "host", "fragment_map_check.cpp")])
    res = subprocess.run([str(exe)], stdout=subprocess.PIPE, text=True)
    assert res.returncode == 0, res.stdout
    assert "fragment maps OK" in res.stdout
