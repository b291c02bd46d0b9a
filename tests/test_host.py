"""Host-side logic that needs no GPU: the C-ABI library loads and exports every symbol the header
declares, argument validation raises RuntimeError for the conditions the reference rejects, the
op schemas match the reference's, pack_scales_blocked matches the oracle's layout."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from prime_moe import _native
    # the seam (prime_moe_hip.h) and the profiling / test hooks (prime_moe_hip_debug.h)
    inc = os.path.join(ROOT, "include")
    header = "".join(open(os.path.join(inc, f)).read() for f in sorted(os.listdir(inc)) if f.endswith(".h"))
    seam = open(os.path.join(inc, "prime_moe_hip.h")).read()
    assert "pmoe_set_phase_mask" not in seam and "pmoe_copy_calibration" not in seam
    declared = set(re.findall(r"\b(pmoe_[a-z0-9_]+)\s*\(", header))
    assert declared == set(_native.SIGNATURES), (declared, set(_native.SIGNATURES))
    lib = _native.load()
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.pmoe_version() == 1
    assert lib.pmoe_last_error() == b"" or isinstance(lib.pmoe_last_error(), bytes)


def test_workspace_query_and_c_side_validation_need_no_gpu():
    from prime_moe import _native
    lib = _native.load()
    # bf16: plan (256 B) + run list with its order (20 B per block + 1) + the two tables of row tiles (16 B per block
    # + 1 each) + fp32 partial sums of
    # the deep contraction split when the problem has at most 32 (block, up weight tile) pairs and K >= 2048
    # (8 parts x 32 KB per fragment and weight tile) + inverse of the sorted order (4 B per pair) + y (one row of
    # K bf16 per pair) + act (rows * H bf16), each rounded to 256 B; the same for both values of split
    assert lib.pmoe_fused_moe_bf16_workspace_bytes(256, 4096, 512, 8, 2048, 4, 1) == \
        256 + 3 * 512 + 8 * 4 * 16 * 2 * 32768 + 256 * 4 * 4 + 256 * 4 * 4096 * 2 + 2048 * 256 * 2
    assert lib.pmoe_fused_moe_bf16_workspace_bytes(256, 4096, 512, 8, 2048, 4, 0) == \
        lib.pmoe_fused_moe_bf16_workspace_bytes(256, 4096, 512, 8, 2048, 4, 1)
    # no partial sums are reserved for a problem too large for the deep split
    assert lib.pmoe_fused_moe_bf16_workspace_bytes(4096, 4096, 28672, 8, 9216, 2, 1) == \
        256 + 1536 + 2 * 1280 + 8192 * 4 + 8192 * 4096 * 2 + 9216 * 14336 * 2
    # mxfp8: header (256 B) + row-tile list (8 B per block) + the two work lists (16 B per block and weight tile)
    # + inverse of the sorted order + y + act (rows * H e4m3) + act scales + re-tiled x scales
    assert lib.pmoe_fused_moe_mxfp8_workspace_bytes(64, 7168, 4096, 256, 33024, 8, 1) == \
        256 + 2304 + 258 * 16 * 16 + 115712 + 64 * 8 * 4 + 64 * 8 * 7168 * 2 + 33024 * 2048 + \
        33024 * 64 + 33024 * 224
    # rejected before any HIP call: status 1 and a message
    rc = lib.pmoe_moe_align(None, None, None, None, 8, 2000, 128, 128, 1024, 8, None)
    assert rc == 1 and b"1024 experts" in lib.pmoe_last_error()
    rc = lib.pmoe_fused_moe_bf16(None, None, None, None, None, None, None, None, 2, 16, 4096, 512, 8, 2048,
                                 64, 64, 4, 2, 1, 1, 1, None, 0, None)
    assert rc == 1 and b"block_m=128" in lib.pmoe_last_error()
    rc = lib.pmoe_fused_moe_mxfp8(*([None] * 11), 2, 16, 4096 + 128, 512, 8, 2048, 128, 64, 4, 2, 1, 1, None, 0, None)
    assert rc == 1 and b"multiple of 256" in lib.pmoe_last_error()
    with pytest.raises(RuntimeError, match="multiple of 256"):
        _native.check(rc)
    # limits of the kernels' own encodings: expert number in 10 bits, 32-bit byte offsets into x
    rc = lib.pmoe_fused_moe_bf16(None, None, None, None, None, None, None, None, 2, 16, 4096, 512, 2000, 2048,
                                 128, 64, 4, 2, 1, 1, 1, None, 0, None)
    assert rc == 1 and b"at most 1024 experts" in lib.pmoe_last_error()
    rc = lib.pmoe_fused_moe_bf16(None, None, None, None, None, None, None, None, 2, 1 << 20, 4096, 512, 8, 2048,
                                 128, 64, 4, 2, 1, 1, 1, None, 0, None)
    assert rc == 1 and b"smaller than 4 GiB" in lib.pmoe_last_error()
    rc = lib.pmoe_fused_moe_mxfp8(*([None] * 11), 2, 1 << 20, 4096, 512, 8, 2048, 128, 64, 4, 2, 1, 1, None, 0, None)
    assert rc == 1 and b"smaller than 4 GiB" in lib.pmoe_last_error()


def test_missing_library_fails_loudly(monkeypatch):
    from prime_moe import _native
    monkeypatch.setattr(_native, "_lib", None)
    monkeypatch.setattr(_native, "LIB_PATH", "/nonexistent/libprime_moe_hip.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        _native.load()


def test_schemas_match_reference_surface():
    import prime_moe  # noqa: F401
    s = str(torch.ops.prime_moe.fused_moe_bf16.default._schema)
    assert s == ("prime_moe::fused_moe_bf16(Tensor x, Tensor w, Tensor w2, Tensor sorted_token_ids, Tensor expert_ids, "
                 "Tensor num_tokens_post_padded, Tensor topk_weights, Tensor(a!) out, int top_k, int block_m, "
                 "int block_n, int warp_n, int stages, int bpc, int cpc, bool split=True) -> ()")
    s = str(torch.ops.prime_moe.fused_moe_mxfp8.default._schema)
    assert s == ("prime_moe::fused_moe_mxfp8(Tensor x, Tensor x_scales, Tensor w, Tensor w_scales, Tensor w2, "
                 "Tensor w2_scales, Tensor sorted_token_ids, Tensor expert_ids, Tensor num_tokens_post_padded, "
                 "Tensor topk_weights, Tensor(a!) out, int top_k, int block_m, int block_n, int warp_n, "
                 "int stages, int bpc, bool split=True) -> ()")
    s = str(torch.ops.prime_moe.moe_align.default._schema)
    assert s == "prime_moe::moe_align(Tensor topk_ids, int num_experts, int block_m, int bpc) -> (Tensor, Tensor, Tensor)"
    assert prime_moe.BLOCK == 32
    assert set(prime_moe.__all__) >= {"fused_moe_bf16", "fused_moe_mxfp8", "pack_scales_blocked", "BLOCK"}


def test_fake_impls_trace_on_meta():
    import prime_moe  # noqa: F401
    ids = torch.empty((64, 8), dtype=torch.int32, device="meta")
    s, e, t = torch.ops.prime_moe.moe_align(ids, 256, 128, 1)
    n = 512
    max_padded = (n + 256 * 127 + 127) // 128 * 128
    assert s.shape == (max_padded,) and e.shape == (max_padded // 128,) and t.shape == (1,)
    x = torch.empty((64, 256), dtype=torch.bfloat16, device="meta")
    w = torch.empty((256, 512, 256), dtype=torch.bfloat16, device="meta")
    w2 = torch.empty((256, 256, 256), dtype=torch.bfloat16, device="meta")
    tw = torch.empty((64, 8), dtype=torch.float32, device="meta")
    assert torch.ops.prime_moe.fused_moe_bf16(x, w, w2, s, e, t, tw, x, 8, 128, 64, 4, 2, 1, 1, True) is None


def test_pack_scales_blocked_matches_oracle_layout():
    import prime_moe
    rng = np.random.default_rng(0)
    s = rng.integers(0, 255, size=(3, 256, 12), dtype=np.uint8)
    got = prime_moe.pack_scales_blocked(torch.from_numpy(s).view(torch.float8_e8m0fnu))
    assert got.dtype == torch.float8_e8m0fnu and got.shape == (3, 256 * 12)
    np.testing.assert_array_equal(got.view(torch.uint8).numpy(), O.pack_scales_blocked(s))
    with pytest.raises(AssertionError):
        prime_moe.pack_scales_blocked(torch.zeros((100, 4), dtype=torch.uint8))
    with pytest.raises(AssertionError):
        prime_moe.pack_scales_blocked(torch.zeros((128, 6), dtype=torch.uint8))


def _bf16_args(T=16, K=256, E=2, N=256, top_k=2):
    x = torch.zeros((T, K), dtype=torch.bfloat16)
    w = torch.zeros((E, N, K), dtype=torch.bfloat16)
    w2 = torch.zeros((E, K, N // 2), dtype=torch.bfloat16)
    s = torch.zeros((E * 128,), dtype=torch.int32)
    e = torch.zeros((E,), dtype=torch.int32)
    t = torch.zeros((1,), dtype=torch.int32)
    tw = torch.zeros((T, top_k), dtype=torch.float32)
    out = torch.zeros((T, K), dtype=torch.bfloat16)
    return [x, w, w2, s, e, t, tw, out, top_k, 128, 64, 4, 2, 1, 1, True]


def test_bf16_validation_matrix():
    # conditions of the reference's TORCH_CHECKs (torch_interface.cpp:132-155)
    import prime_moe
    v = lambda *a: prime_moe._validate_bf16(*a, placement=False)  # CPU tensors: no device checks here
    v(*_bf16_args())
    with pytest.raises(RuntimeError, match="must be a GPU tensor"):
        prime_moe._validate_bf16(*_bf16_args())  # as the op calls it: a CPU tensor never reaches a kernel
    def bad(idx, val):
        a = _bf16_args()
        a[idx] = val
        with pytest.raises(RuntimeError):
            v(*a)
    bad(9, 64)                       # block_m
    bad(10, 32)                      # (block_n, warp_n) = (32, 4)
    bad(12, 0); bad(12, 6)           # stages
    bad(13, 2); bad(14, 2)           # bpc, cpc
    a = _bf16_args(); a[12] = 5
    with pytest.raises(RuntimeError, match="stages<=4"):
        v(*a)
    a[15] = False
    v(*a)                            # stages = 5 is fine without split
    bad(0, torch.zeros((16, 256), dtype=torch.float16))
    bad(0, torch.zeros((16, 192), dtype=torch.bfloat16))         # K % 128 and K mismatch
    bad(0, torch.zeros((0, 256), dtype=torch.bfloat16))
    bad(0, torch.zeros((256, 16), dtype=torch.bfloat16).t())      # not contiguous
    bad(3, torch.zeros((256,), dtype=torch.int64))
    bad(6, torch.zeros((16, 2), dtype=torch.float64))
    bad(7, torch.zeros((16, 256), dtype=torch.float32))
    a = _bf16_args(K=384)            # K % 128 == 0 but not % 256 is allowed on the bf16 path
    v(*a)


def test_mxfp8_validation_matrix():
    # conditions of torch_interface.cpp:208-241
    import prime_moe
    T, K, E, N, top_k = 16, 256, 2, 256, 2
    f8, e8 = torch.float8_e4m3fn, torch.float8_e8m0fnu
    def args():
        return dict(
            x=torch.zeros((T, K), dtype=f8), x_scales=torch.zeros((T, K // 32), dtype=e8),
            w=torch.zeros((E, N, K), dtype=f8), w_scales=torch.zeros((E, N, K // 32), dtype=e8),
            w2=torch.zeros((E, K, N // 2), dtype=f8), w2_scales=torch.zeros((E * K * (N // 2) // 32,), dtype=e8),
            sorted_token_ids=torch.zeros((E * 128,), dtype=torch.int32), expert_ids=torch.zeros((E,), dtype=torch.int32),
            num_tokens_post_padded=torch.zeros((1,), dtype=torch.int32),
            topk_weights=torch.zeros((T, top_k), dtype=torch.float32), out=torch.zeros((T, K), dtype=torch.bfloat16),
            top_k=top_k, block_m=128, block_n=32, warp_n=8, stages=4, bpc=1, split=True)
    prime_moe._validate_mxfp8(**args(), placement=False)  # CPU tensors: no device checks here
    with pytest.raises(RuntimeError, match="must be a GPU tensor"):
        prime_moe._validate_mxfp8(**args())
    for key, val in [("block_m", 64), ("stages", 5), ("stages", 0), ("bpc", 2), ("warp_n", 4),
                     ("x", torch.zeros((T, K), dtype=torch.uint8)),
                     ("x_scales", torch.zeros((T, K // 32), dtype=torch.uint8)),
                     ("x_scales", torch.zeros((T, K // 32 - 1), dtype=e8)),
                     ("w_scales", torch.zeros((E, N, K // 32 + 1), dtype=e8)),
                     ("w2", torch.zeros((E, K, N // 2 + 32), dtype=f8)),
                     ("out", torch.zeros((T, K), dtype=torch.float32)),
                     ("x", torch.zeros((T, K + 128), dtype=f8))]:
        a = args()
        a[key] = val
        with pytest.raises(RuntimeError):
            prime_moe._validate_mxfp8(**a, placement=False)


def test_align_validation_and_sizes():
    import prime_moe
    assert prime_moe.align_sizes(512, 256, 128, 1) == (128, 33024, 258)
    assert prime_moe.align_sizes(65536, 128, 128, 1) == (128, 81792, 639)
    assert prime_moe.align_sizes(10, 3, 24, 3) == (72, 288, 12)
    assert prime_moe.align_sizes(10, 3, 24, 3)[1:] == O.moe_align_sizes(10, 3, 24, 3)[1:]
    ok = torch.zeros((8,), dtype=torch.int32)
    prime_moe._validate_align(ok, 4, 128, 1, placement=False)
    with pytest.raises(RuntimeError, match="must be a GPU tensor"):
        prime_moe._validate_align(ok, 4, 128, 1)
    for a in [(ok.long(), 4, 128, 1), (ok, 0, 128, 1), (ok, 4, 0, 1), (ok, 4, 128, 0), (ok, 1025, 128, 1),
              (torch.zeros((8, 2), dtype=torch.int32)[:, 0], 4, 128, 1)]:
        with pytest.raises(RuntimeError):
            prime_moe._validate_align(*a, placement=False)


def test_ops_refuse_cpu_tensors():
    import prime_moe
    with pytest.raises((NotImplementedError, RuntimeError)):
        prime_moe.fused_moe_bf16(*_bf16_args())


def test_workload_table_matches_benchmark_configs():
    from prime_moe.workloads import CONFIGS
    c = CONFIGS["c2_mixtral_bf16"]
    assert (c.T, c.K, c.E, c.N, c.top_k) == (4096, 4096, 8, 28672, 2) and c.flops == O.approx_flops(4096, 2, 4096, 28672)
    assert round(CONFIGS["c1_readme_bf16"].flops / 1e9, 2) == 6.44
    assert round(CONFIGS["c3_qwen3_bf16"].flops / 1e9, 1) == 618.5
    assert round(CONFIGS["c5_decode_mxfp8"].flops / 1e9, 1) == 45.1
    c4 = CONFIGS["c4_dsv3_mxfp8"]
    assert c4.weight_bytes_per_expert() == (4096 * 7168 + 7168 * 2048) * 33 // 32


def test_sweep_routing_and_columns_on_the_host():
    # the benchmark harness's routing generator (reference: benchmark/benchmark.py:116-121) and its CSV
    # header (benchmark.py:523-543) need no GPU
    from prime_moe import sweep
    g = torch.Generator().manual_seed(0)
    assert int(sweep.generate_topk_ids(16, 2048, 4, 0.0, g).max()) == 0
    ids = sweep.generate_topk_ids(16, 2048, 4, 0.5, g)
    assert ids.dtype == torch.int32 and ids.shape == (2048, 4) and 0 <= int(ids.min()) and int(ids.max()) < 16
    assert 0.47 < float((ids == 0).float().mean()) < 0.60  # 0.5 + 0.5 / 16
    assert sweep.COLUMNS[:6] == ["dtype", "tokens", "E", "K", "N", "top_k"]
    assert sweep.COLUMNS[6:19] == ["naive_ms", "baseline_ms", "noreq_ms", "fused_ms", "speedup", "speedup_noreq",
                                   "speedup_naive", "naive_tflops", "baseline_tflops", "fused_tflops", "max_abs", "rel",
                                   "naive_max_abs"]


def test_no_compiler_use_of_m0_in_kernels_with_direct_to_lds_copies(tmp_path):
    """The copy primitives of csrc/moe_ring.h set M0 inside inline assembly without telling the compiler.  Enforced
    here: in the device assembly of every translation unit that includes them, a kernel that contains such a copy
    names M0 only between the markers of those statements, and the sources use none of the builtins that would
    make the compiler hold a value in M0."""
    import glob
    import re
    import subprocess
    from prime_moe import build
    csrc = build.CSRC
    users = [f for f in glob.glob(os.path.join(csrc, "*.hip")) if "moe_ring.h" in open(f).read() or "moe_tall.h" in open(f).read()]
    assert len(users) == 2, users
    banned = re.compile(r"__builtin_amdgcn_(global_load_lds|raw_buffer_load_lds|struct_buffer_load_lds|ds_gws\w*|s_sendmsg\w*|"
                        r"s_movrel\w*|mov_dpp8)")
    for f in users + [os.path.join(csrc, h) for h in ("moe_ring.h", "moe_tall.h", "moe_tile.h", "moe_pipeline.h")]:
        text = re.sub(r"//[^\n]*", "", open(f).read())  # (the header's comment names them)
        assert not banned.search(text), (f, banned.search(text).group(0))
    for f in users:
        asm = tmp_path / (os.path.basename(f) + ".s")
        cmd = [build.hipcc(), f"--offload-arch={build.ARCH}", "-O3", "-std=c++17", "-munsafe-fp-atomics", *build.DEVICE_FLAGS,
               "-S", "--cuda-device-only", f, "-o", str(asm)]
        res = subprocess.run(cmd, capture_output=True, text=True)
        assert res.returncode == 0, res.stderr[-2000:]
        kernel, in_asm, copies, stray = None, False, {}, {}
        for line in open(asm):
            m = re.match(r"^(_Z\w+):", line)
            if m:
                kernel = m.group(1)
            if ";;#ASMSTART" in line:
                in_asm = True
            elif ";;#ASMEND" in line:
                in_asm = False
            code = line.split(";")[0]
            if kernel is None or not code.strip() or code.lstrip().startswith("."):
                continue
            if "global_load_lds" in code:
                assert in_asm, (kernel, line)  # only the hand-issued ones exist
                copies[kernel] = copies.get(kernel, 0) + 1
            if re.search(r"\bm0\b", code) and not in_asm:
                stray.setdefault(kernel, []).append(line.strip())
        assert copies, f"{f}: no direct-to-LDS copy found in the assembly"
        for k in copies:
            assert k not in stray, (k, stray[k][:5])
