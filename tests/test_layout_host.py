"""Host-side check of the bit layout the MFMA GEMV relies on (compiled with g++, no GPU)."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_decode_layout_matches_activation_image(tmp_path):
    exe = tmp_path / "layout_check"
    subprocess.run(["g++", "-O1", "-std=c++17", "-I", os.path.join(ROOT, "ternary-llm_amd", "csrc"),
                    os.path.join(ROOT, "tests", "layout_check.cpp"), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0 and "bad=0" in out.stdout, out.stdout + out.stderr
