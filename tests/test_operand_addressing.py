"""The kernels' own address arithmetic on the CPU.  tests/addressing_check.cpp includes the header
the GEMM kernels compile for their operand offsets (marian-dev_amd/csrc/operand_addressing.h: lane
columns and their clamps, sub-step clamps, the LDS staging offsets of the large-M tiles, the
detours of a 64-column last K block, shortlist gathers) and walks every lane, wave, tile and K
step of edge shapes - N = 8 / 24 / 1000 / 1032, K = 64 / 192 / 576 / 1088 / 1024, M = 129 ... 300,
shortlists of 8 - through it: every 16-byte load inside its operand, every multiplied chunk
fetched exactly once.  Built with the host sanitizers."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "marian-dev_amd", "csrc")


def test_every_operand_load_stays_inside(tmp_path):
    exe = str(tmp_path / "addressing_check")
    subprocess.check_call(["g++", "-O2", "-std=c++17", "-Wall", "-Werror", "-fsanitize=address,undefined",
                           "-static-libasan", "-static-libubsan", "-I", CSRC, "-o", exe,
                           os.path.join(ROOT, "tests", "addressing_check.cpp")])
    r = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert r.stdout.strip().endswith("ok"), r.stdout


def test_kernels_use_the_checked_helpers():
    """The offsets the check walks are the ones the kernels compute: each kernel source calls the helpers."""
    uses = {
        "gemm_stream32_kernel.h": ["stream32_lane_column(", "stream32_lane_offset(", "stream32_chunk_is_whole(", "stream32_clamped_substep("],
        "gemm_stream_kernel.h": ["stream16_lane_offset("],
        "gemm_mfma32_kernel.h": ["stage_a_offset(", "stage_b_column(", "stage_b_offset(", "stage_a_tail_adjust(", "stage_b_goes_back("],
        "gemm_pair_kernel.h": ["stage_a_row(", "stage_a_chunk(", "stage_b_offset("],
        "decode_ops.hip": ["stream32_lane_offset(", "stream32_clamped_substep(", "proj_row_plan(", "proj_row_of(", "proj_first_sentence("],
    }
    for name, calls in uses.items():
        text = open(os.path.join(CSRC, name)).read()
        for c in calls:
            assert c in text, (name, c)
