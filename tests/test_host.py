"""CPU tests of the host side: the C ABI library loads and exports what the
header declares, argument validation returns the documented codes before any
launch, and the extension raises RuntimeError like the reference's TORCH_CHECKs
(kernel/fused_mha_api.cpp:25-47).  No compute call is made here."""
import ctypes
import inspect
import os
import sys

import pytest
import torch

import abi


ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    return abi.load()


def test_exports_every_declared_symbol(lib):
    names = abi.declared_symbols()
    assert names == sorted(["fused_mha_forward", "fused_mha_backward", "fused_mha_backward_workspace_bytes",
                            "fused_mha_backward_min_workspace_bytes",
                            "fused_mha_backward_noalloc", "fused_mha_backward_delta", "fused_mha_backward_dq", "fused_mha_backward_dkdv",
                            "fused_mha_forward_strided", "fused_mha_backward_strided", "fused_mha_error_string"])
    for name in names:
        assert hasattr(lib, name), name


def test_error_strings(lib):
    seen = set()
    for code in range(0, -11, -1):
        text = lib.fused_mha_error_string(code).decode()
        assert text and text not in seen
        seen.add(text)
    assert b"unknown" in lib.fused_mha_error_string(-99)


def test_workspace_bytes(lib):
    small = lib.fused_mha_backward_min_workspace_bytes
    assert small(2, 32, 4096, 128) == 2 * 2 * 32 * 4096 * 4
    assert small(1, 4, 128, 64) == 2 * 4 * 128 * 4
    assert small(1, 4, 100, 64) == 2 * 4 * 100 * 4  # any n > 0 is accepted
    assert small(1, 4, 0, 64) == 0
    assert small(1, 4, 128, 96) == 0
    # the preferred workspace adds room for the fp16 dS tiles: slices * np * np elements, np = n rounded up to
    # 128, behind the statistics rounded up to 256 bytes
    big = lib.fused_mha_backward_workspace_bytes
    assert big(2, 32, 4096, 128) == 2 * 2 * 32 * 4096 * 4 + 64 * 4096 * 4096 * 2
    assert big(1, 4, 100, 64) == 3328 + 4 * 128 * 128 * 2  # 3200 bytes of statistics -> 3328
    assert big(1, 4, 0, 64) == 0 and big(1, 4, 128, 96) == 0
    # past the spill limit (16 GiB) only the statistics are asked for
    assert big(1, 32, 16384, 128) == small(1, 32, 16384, 128) + 32 * 16384 * 16384 * 2  # 16 GiB: still spilled
    assert big(1, 64, 16384, 128) == small(1, 64, 16384, 128)                           # 32 GiB: recompute path


def test_forward_validation_codes(lib):
    p = 0x1000  # never dereferenced: every call below is rejected before a launch
    f = lib.fused_mha_forward
    assert f(None, p, p, p, p, 1, 1, 32, 32, 64, 1.0, 0, None) == abi.ERR_NULL_POINTER
    assert f(p, p, p, p, None, 1, 1, 32, 32, 64, 1.0, 0, None) == abi.ERR_NULL_POINTER
    assert f(p, p, p, p, p, 0, 1, 32, 32, 64, 1.0, 0, None) == abi.ERR_BAD_SHAPE
    assert f(p, p, p, p, p, 1, 1, 0, 0, 64, 1.0, 0, None) == abi.ERR_BAD_SHAPE        # n == 0
    assert f(p, p, p, p, p, 1, 1, 32, 64, 64, 1.0, 0, None) == abi.ERR_BAD_SHAPE      # m != n
    assert f(p, p, p, p, p, 1, 1, 32, 32, 96, 1.0, 0, None) == abi.ERR_BAD_HEAD_DIM
    assert f(p, p, p, p, p, 1, 1, 32, 32, 64, float("nan"), 0, None) == abi.ERR_BAD_SCALE
    assert f(p, p, p, p, p, 1, 1, 32, 32, 64, float("inf"), 0, None) == abi.ERR_BAD_SCALE
    assert f(p + 2, p, p, p, p, 1, 1, 32, 32, 64, 1.0, 0, None) == abi.ERR_MISALIGNED
    # the limits of the kernels' 32-bit arithmetic and of a launch: n < 2^29, head*d < 2^24,
    # ceil(n/128)*batch*head < 2^23, batch*head*n*d/8 < 2^32
    assert f(p, p, p, p, p, 1, 1, 1 << 29, 1 << 29, 64, 1.0, 0, None) == abi.ERR_TOO_LARGE
    assert f(p, p, p, p, p, 1 << 12, 1 << 12, 1 << 14, 1 << 14, 64, 1.0, 0, None) == abi.ERR_TOO_LARGE
    assert f(p, p, p, p, p, 2048, 2048, 1 << 16, 1 << 16, 64, 1.0, 0, None) == abi.ERR_TOO_LARGE
    assert f(p, p, p, p, p, 1, 1 << 17, 128, 128, 128, 1.0, 0, None) == abi.ERR_TOO_LARGE    # head*d = 2^24
    assert f(p, p, p, p, p, 1, 1 << 18, 128, 128, 64, 1.0, 0, None) == abi.ERR_TOO_LARGE     # head*d = 2^24
    assert f(p, p, p, p, p, 1 << 11, 1 << 12, 128, 128, 64, 1.0, 0, None) == abi.ERR_TOO_LARGE  # 2^23 blocks of 128 rows
    assert f(p, p, p, p, p, 1 << 9, 1 << 12, 130, 130, 128, 1.0, 0, None) == abi.ERR_TOO_LARGE  # delta pass: 2^32 threads
    assert lib.fused_mha_backward_workspace_bytes(1, 1 << 17, 128, 128) == 0
    assert lib.fused_mha_backward_min_workspace_bytes(1, 1 << 17, 128, 128) == 0


def test_backward_validation_codes(lib):
    p = 0x1000
    b = lib.fused_mha_backward
    ws = 2 * 1 * 1 * 32 * 4
    assert b(p, p, p, p, p, p, None, ws, p, p, p, 1, 1, 32, 32, 64, 1.0, 0, None) == abi.ERR_NULL_POINTER
    assert b(p, p, p, p, p, p, p, ws, p, p, None, 1, 1, 32, 32, 64, 1.0, 0, None) == abi.ERR_NULL_POINTER
    assert b(p, p, p, p, p, p, p, ws - 1, p, p, p, 1, 1, 32, 32, 64, 1.0, 0, None) == abi.ERR_BAD_SHAPE
    assert b(p, p, p, p, p, p, p, ws, p, p, p, 1, 1, 40, 40, 64, 1.0, 0, None) == abi.ERR_BAD_SHAPE
    assert b(p, p, p, p, p, p, p, ws, p, p, p, 1, 1, 32, 32, 32, 1.0, 0, None) == abi.ERR_BAD_HEAD_DIM
    assert b(p, p, p, p, p, p, p, ws, p, p + 8, p, 1, 1, 32, 32, 64, 1.0, 0, None) == abi.ERR_MISALIGNED
    assert lib.fused_mha_backward_delta(p, None, p, p, ws, 1, 1, 32, 64, None) == abi.ERR_NULL_POINTER
    assert lib.fused_mha_backward_dq(p, p, p, p, p, p, ws, None, 1, 1, 32, 64, 1.0, 0, None) == abi.ERR_NULL_POINTER
    assert lib.fused_mha_backward_dkdv(p, p, p, p, p, p, ws, p, None, 1, 1, 32, 64, 1.0, 0, None) == abi.ERR_NULL_POINTER


def test_noalloc_validation_codes(lib):
    """Rejected before the scratch address is looked up or anything is launched."""
    p = 0x1000
    g = lib.fused_mha_backward_noalloc
    assert g(p, p, p, p, p, p, p, p, p, 1, 1, 40, 32, 64, 1.0, 0, None) == abi.ERR_BAD_SHAPE
    assert g(p, p, p, p, p, p, p, p, p, 1, 1, 32, 32, 96, 1.0, 0, None) == abi.ERR_BAD_HEAD_DIM
    rows = abi.NOALLOC_MAX_ROWS
    assert g(p, p, p, p, p, p, p, p, p, 1, 2, rows // 2 + 1, rows // 2 + 1, 64, 1.0, 0, None) == abi.ERR_SCRATCH_LIMIT
    assert g(p, p, p, p, p, p, p, p, p, 4, 64, 8192, 8192, 128, 1.0, 1, None) == abi.ERR_SCRATCH_LIMIT
    assert b"NOALLOC_MAX_ROWS" in lib.fused_mha_error_string(abi.ERR_SCRATCH_LIMIT)
    import re
    text = open(abi.HEADER).read()
    assert int(re.search(r"#define FUSED_MHA_NOALLOC_MAX_ROWS \(1 << (\d+)\)", text).group(1)) == 20


def test_strided_validation_codes(lib):
    p = 0x1000  # never dereferenced: every call below is rejected before a launch
    f = lib.fused_mha_forward_strided
    ok = abi.Strides(32 * 2 * 64, 2 * 64, 64)

    def call(qs, ks=ok, vs=ok):
        return f(p, qs, p, ks, p, vs, p, p, 1, 2, 32, 64, 1.0, 0, None)

    assert call(abi.Strides(32 * 2 * 64, 2 * 64, 68)) == abi.ERR_BAD_STRIDE      # rows off 16-byte boundaries
    assert call(ok, abi.Strides(-4096, 128, 64)) == abi.ERR_BAD_STRIDE           # negative
    assert call(ok, ok, abi.Strides(1 << 30, 1 << 24, 64)) == abi.ERR_BAD_STRIDE  # sequence stride too large
    assert f(None, ok, p, ok, p, ok, p, p, 1, 2, 32, 64, 1.0, 0, None) == abi.ERR_NULL_POINTER
    assert f(p, ok, p, ok, p, ok, p, p, 1, 2, 32, 96, 1.0, 0, None) == abi.ERR_BAD_HEAD_DIM
    g = lib.fused_mha_backward_strided
    bad = abi.Strides(4096, 130, 64)
    assert g(p, ok, p, ok, p, ok, p, p, bad, p, p, 1 << 20, p, p, p, 1, 2, 32, 64, 1.0, 0, None) == abi.ERR_BAD_STRIDE
    assert g(p, ok, p, ok, p, ok, p, p, ok, p, p, 8, p, p, p, 1, 2, 32, 64, 1.0, 0, None) == abi.ERR_BAD_SHAPE  # workspace
    assert b"stride" in lib.fused_mha_error_string(abi.ERR_BAD_STRIDE)


def test_python_api_signature():
    import flash_attn_v100
    from flash_attn_v100 import flash_attn_func
    from flash_attn_v100.flash_attn_interface import FlashAttnFunc

    assert flash_attn_v100.__version__
    params = inspect.signature(flash_attn_func).parameters
    # reference flash_attn_interface.py:101-107
    assert list(params) == ["q", "k", "v", "softmax_scale", "causal"]
    assert params["softmax_scale"].default is None and params["causal"].default is False
    assert issubclass(FlashAttnFunc, torch.autograd.Function)


def test_extension_checks_raise_runtime_error():
    import flash_attn_v100_cuda as ext

    def t(*shape, dtype=torch.float16):
        return torch.zeros(shape, dtype=dtype)

    ok = t(1, 32, 2, 64)
    cases = [
        ((t(1, 32, 2, 64, dtype=torch.float32), ok, ok), "fp16"),
        ((ok, t(1, 32, 2, 64, dtype=torch.bfloat16), ok), "same dtype"),
        ((t(32, 2, 64), ok, ok), "4 dimensions"),
        ((t(1, 32, 2, 96), t(1, 32, 2, 96), t(1, 32, 2, 96)), "head dimension"),
        ((t(1, 0, 2, 64), t(1, 0, 2, 64), t(1, 0, 2, 64)), "seqlen must be positive"),
        ((ok, t(1, 64, 2, 64), ok), "must have shape"),
        ((t(1, 32, 2, 128)[..., ::2], ok, ok), "contiguous last dimension"),
        ((ok, ok, ok), "must be on the GPU"),
    ]
    for (q, k, v), msg in cases:
        with pytest.raises(RuntimeError, match=msg):
            ext.fwd(q, k, v, None, 0.125, False)
    lse = torch.zeros(1, 2, 32)
    with pytest.raises(RuntimeError, match="must be on the GPU"):
        ext.bwd(ok, ok, ok, ok, ok, lse, None, None, None, 0.125, True)
    with pytest.raises(RuntimeError, match="lse must be fp32"):
        ext.bwd(ok, ok, ok, ok, ok, lse.half(), None, None, None, 0.125, True)
    with pytest.raises(RuntimeError, match="must have shape"):
        ext.bwd(ok, ok, ok, ok, ok, torch.zeros(1, 32, 2), None, None, None, 0.125, True)
    with pytest.raises(RuntimeError, match="4 dimensions"):
        ext.bwd(ok, ok, t(32, 2, 64), ok, ok, lse, None, None, None, 0.125, True)
    with pytest.raises(RuntimeError, match="4 dimensions"):
        ext.bwd(ok, ok, ok, t(32, 2, 64), ok, lse, None, None, None, 0.125, True)
    with pytest.raises(RuntimeError, match="4 dimensions"):
        ext.bwd(t(2, 64), ok, ok, ok, ok, lse, None, None, None, 0.125, True)


def test_python_api_rejects_cpu_tensors():
    from flash_attn_v100 import flash_attn_func

    q = torch.zeros(1, 32, 2, 64, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="must be on the GPU"):
        flash_attn_func(q, q, q, None, True)


def test_block_map_is_a_bijection(tmp_path):
    """csrc/block_map.h, compiled for the host: every (slice, block) pair is produced exactly once for any slice
    count (multiples of 8 or not), and with a multiple of 8 every slice stays on one XCD (work-group id mod 8)."""
    import os
    import subprocess

    src = tmp_path / "check_block_map.cpp"
    src.write_text(r'''
#include <cstdio>
#include <vector>
#include "block_map.h"
int main() {
  for (int slices = 1; slices <= 83; ++slices)
    for (int bps = 1; bps <= 37; ++bps) {
      const int total = slices * bps;
      std::vector<int> seen(total, 0), xcd_of(slices, -1);
      int shared = 0;
      for (int lin = 0; lin < total; ++lin) {
        int s = -1, b = -1;
        fmha_slice_and_block(lin, slices, bps, s, b);
        if (s < 0 || s >= slices || b < 0 || b >= bps) { printf("range %d %d %d\n", slices, bps, lin); return 1; }
        if (seen[s * bps + b]++) { printf("twice %d %d %d\n", slices, bps, lin); return 1; }
        if (xcd_of[s] < 0) xcd_of[s] = lin & 7;
        else if (xcd_of[s] != (lin & 7) && s < (slices & ~7)) ++shared;
      }
      if (shared) { printf("slice on two XCDs %d %d\n", slices, bps); return 1; }
    }
  // heaviest first inside a slice: block indices of one slice appear in ascending order
  // (the slices beyond a multiple of 8 are cut into per-XCD runs instead)
  for (int slices : {8, 12, 64, 80}) {
    const int bps = 16;
    std::vector<int> last(slices, -1);
    for (int lin = 0; lin < slices * bps; ++lin) {
      int s, b;
      fmha_slice_and_block(lin, slices, bps, s, b);
      if (s < (slices & ~7) && b <= last[s]) { printf("order %d %d\n", slices, lin); return 1; }
      last[s] = b;
    }
  }
  puts("ok");
  return 0;
}
''')
    inc = os.path.join(abi.ROOT, "flash-attention-v100_amd", "csrc")
    exe = tmp_path / "check_block_map"
    subprocess.check_call(["g++", "-O1", "-std=c++17", "-I", inc, str(src), "-o", str(exe)])
    assert subprocess.check_output([str(exe)]).decode().strip() == "ok"


def test_persistent_schedule_covers_every_block_once_and_balances(tmp_path):
    """csrc/block_map.h, compiled for the host: the rounds of the persistent work groups visit every block exactly
    once, a work group's blocks stay on its XCD (block number mod 8), and under causal masking the static
    schedule is balanced: at the headline and the long-context shape no work group gets more than 3 % above the
    mean number of tiles."""
    import os
    import subprocess

    src = tmp_path / "check_persistent.cpp"
    src.write_text(r'''
#include <cstdio>
#include <vector>
#include <algorithm>
#include "block_map.h"
static int check(int total, int G) {
  std::vector<int> seen(total, 0);
  for (int w = 0; w < G; ++w) {
    int r = 0;
    if (fmha_persistent_block(0, w, G) >= total) { printf("first round %d %d %d\n", total, G, w); return 1; }
    int guard = 0;
    while (r >= 0) {
      const int lin = fmha_persistent_block(r, w, G);
      if (lin < 0 || lin >= total) { printf("range %d %d %d %d\n", total, G, w, r); return 1; }
      if ((lin & 7) != (w & 7) && total > G) { printf("xcd %d %d %d %d\n", total, G, w, r); return 1; }
      if (seen[lin]++) { printf("twice %d %d %d\n", total, G, lin); return 1; }
      r = fmha_persistent_next_round(r, w, G, total);
      if (++guard > total + 2) { printf("no end %d %d %d\n", total, G, w); return 1; }
    }
  }
  for (int lin = 0; lin < total; ++lin) if (!seen[lin]) { printf("missed %d %d %d\n", total, G, lin); return 1; }
  return 0;
}
// tiles per work group under causal masking: slices x bps blocks of `rows` queries, 64-key tiles
static double imbalance(int slices, int bps, int rows, int G) {
  const int total = slices * bps;
  std::vector<long> load(G, 0);
  for (int w = 0; w < G; ++w)
    for (int r = 0; r >= 0; r = fmha_persistent_next_round(r, w, G, total)) {
      int s, b;
      fmha_slice_and_block(fmha_persistent_block(r, w, G), slices, bps, s, b);
      const int mblk = bps - 1 - b;  // heavy first
      load[w] += (long)(mblk + 1) * rows / 64;
    }
  long sum = 0, mx = 0;
  for (long v : load) { sum += v; mx = std::max(mx, v); }
  return (double)mx * G / sum;
}
int main() {
  for (int G : {8, 64, 256, 304})
    for (int total = 1; total <= 5 * G + 17; total += (total < 40 ? 1 : 7)) {
      const int grid = total <= G ? total : G;  // what persistent_grid() launches
      if (check(total, grid)) return 1;
    }
  const double head_fwd = imbalance(64, 16, 256, 256), head_dq = imbalance(64, 32, 128, 256);
  const double long_fwd = imbalance(16, 64, 256, 256), long_dq = imbalance(16, 128, 128, 256);
  if (head_fwd > 1.03 || head_dq > 1.03 || long_fwd > 1.03 || long_dq > 1.03) {
    printf("imbalance %.3f %.3f %.3f %.3f\n", head_fwd, head_dq, long_fwd, long_dq);
    return 1;
  }
  puts("ok");
  return 0;
}
''')
    inc = os.path.join(abi.ROOT, "flash-attention-v100_amd", "csrc")
    exe = tmp_path / "check_persistent"
    subprocess.check_call(["g++", "-O1", "-std=c++17", "-I", inc, str(src), "-o", str(exe)])
    assert subprocess.check_output([str(exe)]).decode().strip() == "ok"


def test_installed_distribution_imports_without_pythonpath(tmp_path):
    """`pip install .` (the wheel `python setup.py install` / `pip wheel .` build; reference setup.py:151-172,
    README.md:21-23) puts the package, the extension and the kernel library into one place, and the package
    imports from there with no path into this tree."""
    import os
    import subprocess
    import sys

    pkg = os.path.join(abi.ROOT, "flash-attention-v100_amd")
    target = tmp_path / "site"
    subprocess.check_call([sys.executable, "-m", "pip", "install", "--no-deps", "--no-build-isolation", "--no-index",
                           "--quiet", "--target", str(target), pkg])
    assert (target / "flash_attn_v100_cuda.so").exists()
    assert (target / "flash_attn_v100" / "lib" / "libfused_mha.so").exists()
    code = ("import sys, os; sys.path.insert(0, %r); import flash_attn_v100, flash_attn_v100_cuda; "
            "assert os.path.dirname(flash_attn_v100.__file__).startswith(%r); "
            "assert flash_attn_v100_cuda.__file__.startswith(%r); "
            "print(flash_attn_v100.__version__, callable(flash_attn_v100.flash_attn_func))") % (
                str(target), str(target), str(target))
    env = {k: v for k, v in os.environ.items() if k != "PYTHONPATH"}
    out = subprocess.check_output([sys.executable, "-c", code], cwd=str(tmp_path), env=env).decode()
    assert out.split() == ["0.0.1", "True"]


def test_bench_refuses_more_than_one_gpu():
    """bench.py is a one-GPU benchmark: --gpus N with N > 1 exits with a message that says so."""
    import subprocess

    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr


def test_bench_clock_sampler_helper():
    """The helper bench.py starts for the clock and power sample: parsers on recorded tool output, and the
    one-line-in, one-JSON-line-out protocol (on a machine without the tools the values are null)."""
    import json
    import subprocess

    sys.path.insert(0, ROOT)
    import bench

    text = ("GPU: 0\n    POWER:\n        SOCKET_POWER: 1315 W\n        GFX_VOLTAGE: N/A\n    CLOCK:\n"
            "        GFX_0:\n            CLK: 1885 MHz\n            MIN_CLK: 500 MHz\n            MAX_CLK: 2400 MHz\n"
            "        GFX_1:\n            CLK: 1821 MHz\n            MIN_CLK: 500 MHz\n")
    got = bench.parse_amd_smi(text)
    assert got == {"sclk_mhz": 1853, "socket_power_w": 1315, "xcd_mhz": [1885, 1821]}
    assert bench.parse_amd_smi("no such tool") == {"sclk_mhz": None, "socket_power_w": None, "xcd_mhz": None}
    assert bench.parse_rocm_smi("GPU[0]\t\t: sclk clock level: 1: (1849Mhz)\n") == 1849
    assert bench.parse_rocm_smi("") is None

    p = bench.start_clock_sampler()
    assert p is not None
    p.stdin.write("sample\n")
    p.stdin.flush()
    reply = json.loads(p.stdout.readline())
    assert set(("sclk_mhz", "socket_power_w", "xcd_mhz")) <= set(reply)
    p.stdin.close()
    assert p.wait(timeout=60) == 0


def test_flop_and_byte_counts_of_the_bench():
    sys.path.insert(0, ROOT)
    import bench

    assert bench.fwd_flops(2, 32, 4096, 128, True) == 4 * 2 * 32 * 4096 * 4096 * 128 / 2
    assert bench.fwd_flops(16, 12, 512, 64, False) == 4 * 16 * 12 * 512 * 512 * 64
    fwd_bytes, bwd_bytes = bench.min_hbm_bytes(2, 32, 4096, 128)
    tensor = 2 * 32 * 4096 * 128 * 2
    assert fwd_bytes == 4 * tensor + 2 * 32 * 4096 * 4  # q, k, v, o and lse
    assert bwd_bytes >= 8 * tensor  # q, k, v, o, dO in; dq, dk, dv out
