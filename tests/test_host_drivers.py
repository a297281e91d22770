"""Host drivers: config grammar (CPU) and the result-line format of the executables (GPU)."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def config_check(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("host") / "config_check")
    subprocess.run(["hipcc", "-O1", "-std=c++17", os.path.join(ROOT, "tests", "host", "config_check.cpp"),
                    os.path.join(ROOT, "turbofno_amd", "host", "utils.cpp"), "-o", exe], check=True,
                   stderr=subprocess.DEVNULL)
    return exe


def run_cfg(exe, path):
    return subprocess.run([exe, path], check=True, capture_output=True, text=True).stdout.strip()


def test_config_grammar(config_check, tmp_path):
    # grammar of the reference's benchmark_config/*.txt: "key = v v v", '#' comments, blank lines,
    # last line without trailing newline (utils/utils.cu:14-22, fused.cu:84-90)
    p = tmp_path / "cfg.txt"
    p.write_text("# comment\n\nbs_list = 1 2 4\nDX_list = 128 256\nK_list = 8 16 24 32 40\nN_list = 64")
    assert run_cfg(config_check, str(p)) == "DX_list:128,256;K_list:8,16,24,32,40;N_list:64;bs_list:1,2,4;"
    # a missing file gives zero problems, as in the reference
    assert run_cfg(config_check, str(tmp_path / "missing.txt")) == ""


def test_shipped_configs_parse(config_check):
    out = run_cfg(config_check, os.path.join(ROOT, "benchmark_config", "problem_size_1d.txt"))
    assert "dimX_list:1;" in out and "DY_list:128,256;" in out and "K_list:8,16,24,32;" in out
    out = run_cfg(config_check, os.path.join(ROOT, "benchmark_config", "problem_size_2d.txt"))
    assert "DX_list:128,256;" in out and "bs_list:1,4,16;" in out


@pytest.mark.gpu
def test_driver_result_lines(tmp_path):
    exe1, exe2 = os.path.join(ROOT, "bin", "TurboFNO_1D_D"), os.path.join(ROOT, "bin", "TurboFNO_2D_D")
    assert os.path.exists(exe1) and os.path.exists(exe2), "build the drivers with make -C turbofno_amd/host"
    out = subprocess.run([exe1, "4", "1", "128", "64", "16"], check=True, capture_output=True, text=True, timeout=100).stdout
    print(out, flush=True)
    assert re.fullmatch(r"1D_D, bs=4   , dimX=1   , DY=128 , N=64  , K=16  , TIME=\s*\d+\.\d{3}ms\n", out), out
    out = subprocess.run([exe2, "1", "256", "256", "64", "16"], check=True, capture_output=True, text=True, timeout=100).stdout
    print(out, flush=True)
    assert re.fullmatch(r"2D_D, bs=1   , DX=256 , DY=256 , N=64  , K=16  , TIME=\s*\d+\.\d{3}ms\n", out), out
    # config-file mode: a tiny grid, loop order bs -> DX -> DY -> N -> K
    cfg = str(tmp_path / "tiny_2d.txt")
    with open(cfg, "w") as f:
        f.write("bs_list = 1\nDX_list = 128 256\nDY_list = 128\nN_list = 64\nK_list = 8 16")
    lines = subprocess.run([exe2, cfg], check=True, capture_output=True, text=True, timeout=100).stdout.splitlines()
    got = [tuple(int(v) for v in re.findall(r"=(\d+)", ln)[:5]) for ln in lines]
    assert got == [(1, 128, 128, 64, 8), (1, 128, 128, 64, 16), (1, 256, 128, 64, 8), (1, 256, 128, 64, 16)], lines


def test_driver_refuses_malformed_arguments_before_touching_the_gpu():
    """five positional arguments that are not positive integers end the run with a message (no HIP call has happened
    yet, so this runs without a GPU)"""
    for v in "AD":
        exe = os.path.join(ROOT, "bin", f"TurboFNO_1D_{v}")
        assert os.path.exists(exe), "build the drivers with make -C turbofno_amd/host"
        for bad in (["4", "1", "12x", "64", "16"], ["0", "1", "128", "64", "16"], ["4", "1", "128", "", "16"],
                    ["4", "1", "128", "64", "99999999999"]):
            r = subprocess.run([exe] + bad, capture_output=True, text=True, timeout=100)
            assert r.returncode == 1 and "is not a positive integer" in r.stderr and r.stdout == "", (bad, r)


@pytest.mark.gpu
@pytest.mark.parametrize("variant", "ABCD")
def test_driver_skips_lengths_without_a_kernel(variant, tmp_path):
    """a length that is not 128, 256, 512 or 1024 has no kernel-table entry: every variant prints why and skips the
    problem instead of running a kernel of a neighbouring length on its buffers"""
    cfg = str(tmp_path / "odd_2d.txt")
    with open(cfg, "w") as f:
        f.write("bs_list = 1\nDX_list = 128 200\nDY_list = 128 96\nN_list = 64 96\nK_list = 8")
    exe = os.path.join(ROOT, "bin", f"TurboFNO_2D_{variant}")
    r = subprocess.run([exe, cfg], check=True, capture_output=True, text=True, timeout=100)
    lines = r.stdout.splitlines()
    got = [tuple(int(v) for v in re.findall(r"=(\d+)", ln)[:5]) for ln in lines]
    assert got == [(1, 128, 128, 64, 8)], (lines, r.stderr)
    assert r.stderr.count("problem skipped") == 7, r.stderr


def test_seeded_input_generators(tmp_path):
    """the C++ generators of the benchmark configurations' inputs: ranges, unit variance, smoothness, reproducibility"""
    exe = str(tmp_path / "inputs_check")
    subprocess.run(["g++", "-O2", "-std=c++17", os.path.join(ROOT, "tests", "host", "inputs_check.cpp"),
                    os.path.join(ROOT, "turbofno_amd", "host", "inputs.cpp"), "-o", exe], check=True)
    rows = {ln.split()[0]: [float(v) for v in ln.split()[1:]] for ln in
            subprocess.run([exe], check=True, capture_output=True, text=True).stdout.splitlines()}
    mn, mx, mean, var, low = rows["uniform"]
    assert -1.0 <= mn < -0.99 and 0.99 < mx <= 1.0 and abs(mean) < 0.02 and abs(var - 2.0 / 3.0) < 0.03 and low < 0.7
    mn, mx, mean, var, low = rows["smooth"]
    assert abs(var - 8.0) < 0.5 and low > 0.999                    # eight unit sinusoids per part, all below bin 33
    mn, mx, mean, var, low = rows["vorticity"]
    assert abs(var - 1.0) < 1e-4 and low > 0.99                    # unit variance per channel, red spectrum
    assert rows["reproducible"] == [1.0] and rows["differs"] == [1.0]
    wmax, wvar = rows["weights"]
    assert wmax <= 0.25 + 1e-6 and abs(wvar - 2.0) < 0.2             # uniform / sqrt(16); K * var of complex normal / sqrt(K) = 2


def _run_variant(exe, args, inputs=None):
    env = dict(os.environ, TURBOFNO_DIGEST="1", TURBOFNO_NTEST="2")
    if inputs:
        env["TURBOFNO_INPUTS"] = inputs
    r = subprocess.run([exe] + [str(a) for a in args], check=True, capture_output=True, text=True, timeout=100, env=env)
    digest = [float(v) for v in re.search(r"digest: (\S+) (\S+) (\S+)", r.stderr).groups()]
    return r.stdout, digest


@pytest.mark.gpu
@pytest.mark.parametrize("dim,args", [("1D", (4, 1, 128, 64, 16)), ("1D", (1, 1, 256, 128, 24)),
                                      ("2D", (1, 128, 256, 64, 16)), ("2D", (2, 256, 128, 64, 8)),
                                      ("1D", (2, 1, 1024, 64, 16)), ("2D", (1, 512, 128, 64, 8))])
def test_all_variants_agree(dim, args):
    # with TURBOFNO_DIGEST the ten executables reseed rand() per problem and see identical inputs: the staged (A), half-fused (B, C),
    # fully fused (D) and library (E: hipFFT + hipBLAS) sequences must give the same output up to fp32 rounding.
    # The first launch runs on a zeroed C, so beta does not enter.
    bs, dx, dy, n, k = args
    nelem = bs * dx * dy * n
    xname = "DX" if dim == "2D" else "dimX"
    ref = None
    for v in "ABCDE":
        exe = os.path.join(ROOT, "bin", f"TurboFNO_{dim}_{v}")
        assert os.path.exists(exe), "build the drivers with make -C turbofno_amd/host"
        print(exe, args, flush=True)
        out, dg = _run_variant(exe, args)
        assert re.fullmatch(rf"{dim}_{v}, bs={bs:<4d}, {xname}={dx:<4d}, DY={dy:<4d}, N={n:<4d}, K={k:<4d}, TIME=\s*\d+\.\d{{3}}ms\n", out), out
        assert dg[2] > 0
        if ref is None:
            ref = dg
            continue
        scale = (ref[2] * nelem) ** 0.5          # bound of a weighted sum of nelem terms with that l2
        assert abs(dg[2] - ref[2]) <= 1e-4 * ref[2], (v, dg, ref)
        assert abs(dg[0] - ref[0]) <= 1e-5 * scale and abs(dg[1] - ref[1]) <= 1e-5 * scale, (v, dg, ref)


@pytest.mark.gpu
@pytest.mark.parametrize("dim,args,inputs", [("1D", (8, 1, 256, 128, 64), "smooth"), ("2D", (2, 256, 256, 64, 16), "vorticity"),
                                             ("2D", (1, 128, 128, 64, 16), "uniform")])
def test_variants_agree_on_seeded_inputs(dim, args, inputs):
    """TURBOFNO_INPUTS selects the seeded generators of the benchmark configurations: the fully fused (D) and the library
    (E: hipFFT + hipBLAS) executables must agree on them as well"""
    ref = None
    for v in "DE":
        exe = os.path.join(ROOT, "bin", f"TurboFNO_{dim}_{v}")
        print(exe, args, inputs, flush=True)
        out, dg = _run_variant(exe, args, inputs)
        assert dg[2] > 0
        if ref is None:
            ref = dg
            continue
        nelem = args[0] * args[1] * args[2] * args[3]
        scale = (ref[2] * nelem) ** 0.5
        assert abs(dg[2] - ref[2]) <= 1e-4 * ref[2], (v, dg, ref)
        assert abs(dg[0] - ref[0]) <= 2e-5 * scale and abs(dg[1] - ref[1]) <= 2e-5 * scale, (v, dg, ref)
