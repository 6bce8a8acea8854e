"""The register-FFT engine of the convolution kernel, run on the CPU: the
phases in megalodon_amd/csrc/fftconv_core.hpp are plain C++, so a g++ build
emulates one workgroup (lanes one after another, LDS as an array) and is
checked against numpy's float64 FFT.  Catches index / twiddle mistakes
without a GPU."""
import ctypes
import os
import subprocess

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "native", "fftconv_emu.cc")


@pytest.fixture(scope="module")
def emu(tmp_path_factory):
    out = tmp_path_factory.mktemp("emu") / "libfftconv_emu.so"
    subprocess.run(["g++", "-O1", "-std=c++17", "-shared", "-fPIC", "-o", str(out), SRC], check=True)
    return ctypes.CDLL(str(out))


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


@pytest.mark.parametrize("logm", [11, 12, 13, 14])
@pytest.mark.parametrize("h", [0, 1])
def test_half_transform_matches_numpy_fft(emu, logm, h):
    M = 1 << logm
    rng = np.random.default_rng(logm * 2 + h)
    inr = rng.standard_normal(M).astype(np.float32)
    ini = rng.standard_normal(M).astype(np.float32)
    outr = np.zeros(M, np.float32)
    outi = np.zeros(M, np.float32)
    assert emu.emu_fft_half(logm, h, _p(inr), _p(ini), _p(outr), _p(outi)) == 0
    z = inr.astype(np.float64) + 1j * ini.astype(np.float64)
    if h:
        z = z * np.exp(-2j * np.pi * np.arange(M) / (2 * M))
    want = np.fft.fft(z)
    assert np.abs((outr + 1j * outi) - want).max() / np.abs(want).max() < 2e-6


@pytest.mark.parametrize("logm", [11, 12, 13, 14])
def test_convolution_matches_numpy(emu, logm):
    M = 1 << logm
    rng = np.random.default_rng(logm)
    for L in (2 * M, 2 * M - 1, M + 3):
        for flip_a, flip_out in ((0, 0), (1, 1)):
            a = rng.standard_normal(L).astype(np.float32)
            b = rng.standard_normal(L).astype(np.float32)
            y = np.zeros(L, np.float32)
            assert emu.emu_fftconv(logm, _p(a), _p(b), L, flip_a, flip_out, _p(y)) == 0
            aa = a[::-1] if flip_a else a
            n = 4 * M
            want = np.fft.irfft(np.fft.rfft(aa.astype(np.float64), n) * np.fft.rfft(b.astype(np.float64), n), n)[:L]
            if flip_out:
                want = want[::-1]
            assert np.abs(y - want).max() / np.abs(want).max() < 5e-6
