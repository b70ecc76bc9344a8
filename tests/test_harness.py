"""The process-level harness (morello_amd/mrl_harness) speaks the protocol of a program
Morello emits: one raw little-endian file per parameter in logical row-major order
(verification.rs:76-92, 957-1001), shape line plus elements on stdout (cpu.rs:570-618),
exit status 1 / 2 for bad argument count / unreadable input (cpu.rs:344-364), and
`cpu: <s>s <ns>ns` in benchmark mode (cpu.rs:561-565; parser codegen/mod.rs:358-383)."""
import os
import re
import subprocess

import numpy as np
import pytest

import morello_amd as M
import orc
from morello_amd import synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HARNESS = os.path.join(ROOT, "morello_amd", "mrl_harness")


def run(*args):
    return subprocess.run([HARNESS, *args], capture_output=True, text=True, timeout=120)


def parse_output(text, np_dtype):
    """verification.rs:1003-1051: first line is the shape, `//` lines and blank lines are
    skipped, the rest are whitespace-separated values in logical row-major order."""
    lines = [l for l in text.splitlines() if l.strip() and not l.startswith("//")]
    shape = [int(x) for x in lines[0].split("x")]
    vals = " ".join(lines[1:]).split()
    conv = float if np.issubdtype(np_dtype, np.floating) else int
    return np.array([conv(v) for v in vals], dtype=np_dtype).reshape(shape)


def parse_benchmark_output(text):
    """codegen/mod.rs:358-383: first line `cpu: <s>s <ns>ns`."""
    m = re.fullmatch(r"cpu: (\d+)s (\d+)ns", text.splitlines()[0])
    assert m, text
    return int(m.group(1)) + int(m.group(2)) * 1e-9


def test_argument_and_load_errors(tmp_path):
    assert os.path.exists(HARNESS), "build with python -m morello_amd.build"
    assert run().returncode == 1
    assert run("matmul:1x4x4x4:f32,f32,f32", "a", "b").returncode == 1          # k+1 files needed
    r = run("matmul:1x4x4x4:f32,f32,f32", str(tmp_path / "x"), str(tmp_path / "y"), str(tmp_path / "z"))
    assert r.returncode == 2 and "Error loading input tensors." in r.stderr
    short = tmp_path / "short"
    short.write_bytes(b"\0" * 10)                                                # wrong size
    assert run("matmul:1x4x4x4:f32,f32,f32", str(short), str(short), str(short)).returncode == 2
    assert run("bogus:1x2:f32,f32").returncode == 1
    assert run("matmul:1x4x0x4:f32,f32,f32").returncode == 1
    assert run("matmul:1x4x4x4:f32,f32").returncode == 1
    assert run("softmax:4x4:f32,f32:scan=5").returncode == 1


def test_benchmark_line_parser_cases():
    # the reference's own parser expectations (codegen/mod.rs:389-451)
    assert parse_benchmark_output("cpu: 10s 500ns\n") == pytest.approx(10 + 500e-9)
    assert parse_benchmark_output("cpu: 0s 1000000000ns\n") == pytest.approx(1.0)
    for bad in ("10s 500ns", "cpu: 10 500ns", "cpu: -1s 5ns"):
        with pytest.raises(AssertionError):
            parse_benchmark_output(bad)


@pytest.mark.gpu
def test_check_mode_matmul_reference_inputs(gpu, tmp_path):
    """check_correctness as the reference runs it (verification.rs:863-891): counting inputs
    in every parameter, output file included."""
    shape = [1, 64, 64, 64]
    files = []
    arrs = [synth.check_pattern("u8", (1, 64, 64)), synth.check_pattern("i8", (1, 64, 64)),
            synth.check_pattern("i32", (1, 64, 64))]
    for i, a in enumerate(arrs):
        f = tmp_path / f"p{i}"
        a.tofile(f)
        files.append(str(f))
    r = run("matmul:1x64x64x64:u8,i8,i32:accum", *files)
    assert r.returncode == 0, r.stderr
    assert r.stdout.splitlines()[0] == "1x64x64"
    got = parse_output(r.stdout, np.int32)
    want = orc.matmul(shape, [0, 1, 5], arrs[0], arrs[1], arrs[2].copy(), True)
    assert np.array_equal(got, want)
    # no files: zero-filled buffers (cpu.rs:320) -> all-zero output
    r = run("matmul:1x8x8x8:f32,f32,f32")
    assert r.returncode == 0 and parse_output(r.stdout, np.float32).sum() == 0
    assert "0.0000000000 " in r.stdout                     # %.10f, space after every element


@pytest.mark.gpu
def test_check_mode_other_specs(gpu, tmp_path):
    def files_for(arrs):
        out = []
        for i, a in enumerate(arrs):
            f = tmp_path / f"q{len(os.listdir(tmp_path))}_{i}"
            np.ascontiguousarray(a).tofile(f)
            out.append(str(f))
        return out
    # Softmax, f32 text round trip at %.10f
    x = synth.normal_f32(501, 0, (3, 40))
    r = run("softmax:3x40:f32,f32:scan=1", *files_for([x, np.zeros_like(x)]))
    assert r.returncode == 0, r.stderr
    got = parse_output(r.stdout, np.float32)
    assert np.abs(got - orc.softmax([3, 40], 1, x)).max() < 1e-6   # the reference's own tolerance
    # Conv with NHWC/KRSC Spec layouts: files are logical (NCHW / FCRS) row-major
    shape = [1, 64, 64, 4, 5, 3, 3]
    img = synth.uniform_u8(502, 0, (1, 64, 6, 7))
    filt = synth.uniform_i8(502, 1, (64, 64, 3, 3))
    r = run("conv:1x64x64x4x5x3x3:u8,i8,i32", *files_for([img, filt, np.zeros((1, 64, 4, 5), np.int32)]))
    assert r.returncode == 0, r.stderr
    want = orc.conv(shape, [0, 1, 5], img, filt, np.zeros((1, 64, 4, 5), np.int32))
    assert np.array_equal(parse_output(r.stdout, np.int32), want)
    # Compose with KT given logically ([b,k,n2] row-major file) but laid out k-fastest (bcm)
    b, m, k, n2, n = 1, 128, 128, 128, 128
    q = synth.normal_bf16(503, 0, (b, m, k), 0.5)
    kmat = synth.normal_bf16(503, 1, (b, n2, k), 0.5)
    v = synth.normal_bf16(503, 2, (b, n2, n), 0.5)
    kt = np.ascontiguousarray(kmat.transpose(0, 2, 1))
    r = run("msm:1x128x128x128x128:bf16,bf16,bf16,f32:layouts=rm,rm,bcm,rm",
            *files_for([v, q, kt, np.zeros((b, m, n), np.float32)]))
    assert r.returncode == 0, r.stderr
    want = orc.compose_msm(b, m, k, n2, n, [7, 7, 7, 6], v, q, kt, np.zeros((b, m, n), np.float32))
    got = parse_output(r.stdout, np.float32)
    assert np.abs(got - want).max() / np.abs(want).max() < 1e-2
    # A packed B layout spelled out (layout![0, 2, 1, 2 p(16)], examples/matmul_x86.rs:34-53):
    # the file stays logical row-major, the harness brings it to the layout on the device.
    A, Bm = synth.uniform_u8(505, 0, (1, 8, 32)), synth.uniform_i8(505, 1, (1, 32, 48))
    r = run("matmul:1x8x32x48:u8,i8,i32:layouts=rm,0.2.1.2p16,rm", *files_for([A, Bm, np.zeros((1, 8, 48), np.int32)]))
    assert r.returncode == 0, r.stderr
    assert np.array_equal(parse_output(r.stdout, np.int32),
                          orc.matmul([1, 8, 32, 48], [0, 1, 5], A, Bm, np.zeros((1, 8, 48), np.int32)))
    assert run("matmul:1x8x32x48:u8,i8,i32:layouts=rm,0.2.1.2p7,rm").returncode == 1   # 7 does not divide 48
    # A primitive with two written parameters prints both, in parameter order.
    x = synth.normal_f32(504, 0, (4, 50))
    r = run("softmaxdenominatorandmax:4x50:f32,f32,f32:scan=1",
            *files_for([x, np.zeros((4, 1), np.float32), np.zeros((4, 1), np.float32)]))
    assert r.returncode == 0, r.stderr
    first, second = r.stdout.split("4x1\n")[1:]
    mx = np.array(first.split(), np.float32).reshape(4, 1)
    dn = np.array(second.split(), np.float32).reshape(4, 1)
    wmx, wdn = np.zeros((4, 1), np.float32), np.zeros((4, 1), np.float32)
    orc.softmax_part(orc.PART_DENOM_MAX, (4, 50), 1, [x, wmx, wdn])
    assert np.abs(mx - wmx).max() < 1e-6 and np.abs(dn - wdn).max() / wdn.max() < 1e-5


@pytest.mark.gpu
def test_bench_mode(gpu):
    r = run("matmul:1x1024x1024x1024:u8,i8,i32:accum", "--bench", "20")
    assert r.returncode == 0, r.stderr
    secs = parse_benchmark_output(r.stdout)
    assert 0 < secs < 1.0
