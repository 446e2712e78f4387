"""The harness executables keep the reference program's command line and printouts
(opus_gemm/block_scale_gemm/gemm_a8w8_blockscale_host.cc:128-294)."""
import os
import re
import subprocess

import pytest

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "harness")


def _exe(name):
    path = os.path.join(HERE, name)
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", HERE, name], stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    return path


def _run(name, *argv):
    return subprocess.run([_exe(name), *argv], capture_output=True, text=True, timeout=300)


def test_cli_rejects_like_the_reference():
    r = _run("gemm_a8w8_blockscale.exe", "-m", "0")
    assert r.returncode == 1 and "must be positive" in r.stderr          # host.cc:175-178
    r = _run("gemm_a8w8_blockscale.exe", "-n=100")
    assert r.returncode == 1 and "multiples of GROUP_M/GROUP_N/GROUP_K" in r.stderr   # host.cc:183-187
    r = _run("gemm_a8w8_8wave.exe", "--scale-mode", "bogus")
    assert r.returncode == 1


@pytest.mark.gpu
def test_blockscale_program_default_problem_and_flags():
    r = _run("gemm_a8w8_blockscale.exe", "-v", "1")                      # defaults b=8 m=256 n=512 k=256
    assert r.returncode == 0, r.stdout + r.stderr
    assert "Launching GEMM kernel: M=256, N=512, K=256, grid=(2,1,8), block=512" in r.stdout
    assert r.stdout.count("block_256x256x128] VALID") == 8
    assert "[Overall] ALL BATCHES VALID" in r.stdout
    assert re.search(r"Kernel Performance: avg_time=\d+\.\d{4} ms, \d+\.\d{2} TFlops", r.stdout)
    r = _run("gemm_a8w8_blockscale.exe", "-b=1", "-m=1024", "--n", "1024", "-k", "1024", "--verify=1")
    assert r.returncode == 0 and "[GEMM batch 1/1: 1024x1024x1024, block_256x256x128] VALID" in r.stdout


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["tensor", "rowcol", "mx", "mxt"])
def test_dense_program(mode):
    r = _run("gemm_a8w8_8wave.exe", "-m", "512", "-n", "768", "-k", "512", "-v", "1", "--scale-mode", mode)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "[Overall] ALL BATCHES VALID" in r.stdout and "Kernel Performance:" in r.stdout


@pytest.mark.gpu
def test_flatmm_program():
    r = _run("flatmm_a8w8.exe", "-m", "16", "-n", "2048", "-k", "1024", "-v", "1")
    assert r.returncode == 0, r.stdout + r.stderr
    assert "[Overall] ALL BATCHES VALID" in r.stdout and "Kernel Performance:" in r.stdout


@pytest.mark.gpu
def test_iteration_flags():
    r = _run("gemm_a8w8_8wave.exe", "-m", "256", "-n", "256", "-k", "256", "--iters", "3", "--warmup=2")
    assert r.returncode == 0 and "Kernel Performance:" in r.stdout, r.stdout + r.stderr
    r = _run("gemm_a8w8_8wave.exe", "--iters", "0")
    assert r.returncode == 1 and "--iters must be positive" in r.stderr


@pytest.mark.gpu
def test_buffer_range_check_covers_the_scalar_offset():
    """The kernels move between row groups with the scalar offset of their buffer loads and rely on rows past the
    end of a matrix reading as zero: the hardware's range check has to include that offset (measured on the device,
    every address inside one live allocation)."""
    r = _run("buffer_bounds_probe.exe")
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.count(" ok\n") == 5 and "UNEXPECTED" not in r.stdout
