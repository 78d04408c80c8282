"""GPU parity of the HIP path (through the C ABI) against the CPU oracle.

Bar: int8 activation codes, float32 activation scales and int32 accumulators are
bit-exact; bf16 outputs satisfy |a - b| <= 2e-2 + 1e-2 * |b| elementwise.
"""

import hashlib

import numpy as np
import pytest

from golden import host_case
from oracle import w8a8_oracle as o
import w8a8_cases as wc

pytestmark = pytest.mark.gpu
F32 = np.float32
ATOL, RTOL = 2e-2, 1e-2


@pytest.fixture(scope="module")
def dev():
    torch = pytest.importorskip("torch")
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture(scope="module")
def pkg():
    from __graft_entry__ import load_package

    p = load_package()
    p._native.load()  # fail loudly if the HIP library is missing
    return p


def _assert_integer_stages(aux, st):
    np.testing.assert_array_equal(aux["x_codes"], st["x_codes"])
    np.testing.assert_array_equal(aux["x_scales"].view(np.uint32), st["x_scales"].view(np.uint32))
    np.testing.assert_array_equal(aux["acc"], st["acc"])


def _assert_close(got, want, what=""):
    rep = wc.compare(got, want)
    print(f"[parity]{what} {rep}", flush=True)
    assert rep["violations"] == 0, rep
    # reference gate (relative L2 < 1e-2, cosine >= 0.9999); its max-abs bound of 0.25 presumes
    # O(1) outputs and is reported, not asserted, since one bf16 ulp at magnitude 64 is 0.5
    assert rep["relative_l2"] < 1e-2 and rep["cosine"] >= 0.9999, rep
    return rep


def test_host_case_bitwise(dev, pkg):
    """The reference's SHA-256-pinned case through the reference's own call signature."""
    import torch

    c = host_case.build()
    ql = pkg.quantized_lora
    w = ql.GroupQuantizedWeight(torch.from_numpy(c["weight_codes"]).to(dev),
                                torch.from_numpy(c["weight_scales"]).to(dev).to(torch.bfloat16),
                                64, 64, 8, 64)
    bf = lambda a: torch.from_numpy(a).to(dev).to(torch.bfloat16)
    out = ql.quantized_lora_linear(bf(c["x"]), w, bf(c["lora_a"]), bf(c["lora_b"]), float(c["lora_scaling"]))
    torch.cuda.synchronize()
    got = out.to(torch.float32).cpu().numpy()
    assert got.shape == (3, 32)
    digest = o.sha256_bf16(np.ascontiguousarray(got[:, :17]))
    assert digest == host_case.SPEC["sha256"]["expected"]
    assert np.all(got[:, 17:] == 0)


@pytest.mark.parametrize("m,k,student", [(3, 64, False), (128, 1024, False), (33, 4096, False),
                                         (16, 12288, False), (65, 2560, True), (5, 16384, True), (7, 72, False)])
def test_quantize_rows_bit_exact(dev, pkg, m, k, student):
    import torch

    rng = np.random.default_rng(m * 1000 + k)
    x = rng.standard_t(3, (m, k)) if student else rng.standard_normal((m, k))
    x = o.bf16_round(x.astype(F32))
    x[m // 2] = 0.0                      # an all-zero row: scale 1, codes 0
    if m > 2:
        x[1, :] = o.bf16_round(F32(1e-30))  # tiny but non-zero row
    want_c, want_s = o.quantize_rows(x)
    codes, scales = pkg.w8a8_lora.dynamic_quantize_rows(torch.from_numpy(x).to(dev).to(torch.bfloat16))
    torch.cuda.synchronize()
    np.testing.assert_array_equal(codes.cpu().numpy(), want_c)
    np.testing.assert_array_equal(scales.cpu().numpy().view(np.uint32), want_s.view(np.uint32))


@pytest.mark.parametrize("k,n", [(64, 17), (128, 256), (1024, 3072), (2560, 520)])
def test_pack_unpack_roundtrip(dev, pkg, k, n):
    import torch

    rng = np.random.default_rng(k + n)
    codes = rng.integers(-128, 128, (k, n), dtype=np.int8)
    w = pkg.quantized_lora.GroupQuantizedWeight(torch.from_numpy(codes).to(dev),
                                                torch.ones((1, n), device=dev), k, k, 8, k)
    packed = pkg.w8a8_lora.prepare_weight(w)
    assert packed.packed.numel() == ((k + 127) // 128 * 128) * ((n + 255) // 256 * 256)
    back = pkg.w8a8_lora.unpack_weight(packed)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(back.cpu().numpy(), codes)
    assert pkg.w8a8_lora.prepare_weight(w) is packed  # cached: the permutation is load-time only


def test_config1_single_adapter(dev):
    """benchmark configuration 1: M128 K1024 N3072, one adapter rank 16 alpha 16."""
    case = wc.make_case(128, 1024, 3072, n_adapters=1, rank=16, seed=1, idx_mode="zero")
    st = wc.oracle_forward(case, return_stages=True)
    got, aux = wc.gpu_forward(case)
    _assert_integer_stages(aux, st)
    _assert_close(got, st["out"], " cfg1")


def test_base_only_no_lora(dev):
    case = wc.make_case(70, 256, 300, n_adapters=0, seed=2)
    st = wc.oracle_forward(case, return_stages=True)
    got, aux = wc.gpu_forward(case)
    _assert_integer_stages(aux, st)
    # without LoRA the float32 epilogue has no summation freedom: bit-exact bf16
    np.testing.assert_array_equal(o.bf16_bits(got), o.bf16_bits(st["out"]))


@pytest.mark.parametrize("m,k,n,n_ad,rank", [(512, 512, 1024, 8, 32), (300, 256, 512, 5, 8),
                                             (1000, 384, 768, 64, 16), (64, 128, 256, 3, 64)])
def test_multi_adapter_routing(dev, m, k, n, n_ad, rank):
    case = wc.make_case(m, k, n, n_adapters=n_ad, rank=rank, seed=3 + n_ad)
    case["s"] = np.linspace(0.25, 2.0, n_ad).astype(F32)
    st = wc.oracle_forward(case, return_stages=True)
    got, aux = wc.gpu_forward(case)
    _assert_integer_stages(aux, st)
    _assert_close(got, st["out"], f" multi {m}x{k}x{n} a{n_ad} r{rank}")


@pytest.mark.parametrize("n", [17, 19, 31, 33])
@pytest.mark.parametrize("k", [64, 128])
def test_n_tails_and_row_tail(dev, n, k):
    """Output tails 17/19/31/33 and M = 33 (tests/tx/kernels/rocm/test_w8a8_lora.py:95-124)."""
    case = wc.make_case(33, k, n, n_adapters=1, rank=8, seed=n + k, idx_mode="zero")
    st = wc.oracle_forward(case, return_stages=True)
    got, aux = wc.gpu_forward(case)
    _assert_integer_stages(aux, st)
    _assert_close(got, st["out"], f" tails n{n} k{k}")


def test_rms_gate_up_swiglu_reduced(dev):
    """Config 2 at reduced size: RMSNorm -> gate/up + 8 adapters rank 32 -> SwiGLU."""
    case = wc.make_case(512, 1024, 2048, n_adapters=8, rank=32, seed=5, rms=True, swiglu=True)
    st = wc.oracle_forward(case, return_stages=True)
    got, aux = wc.gpu_forward(case)
    np.testing.assert_array_equal(o.bf16_bits(aux["normalized"]), o.bf16_bits(st["normalized"]))
    _assert_integer_stages(aux, st)
    _assert_close(got, st["out"], " cfg2-reduced")
    # stage-wise: SwiGLU of the GPU's own pre-activation equals the oracle's SwiGLU to 1 bf16 ulp
    case2 = dict(case, swiglu=False)
    fused_gpu, _ = wc.gpu_forward(case2)
    prod_from_gpu_fused = o.swiglu_from_interleaved(fused_gpu)
    d = np.abs(o.bf16_bits(got).astype(np.int32) - o.bf16_bits(prod_from_gpu_fused).astype(np.int32))
    assert d.max() <= 1
    _assert_close(fused_gpu, st["fused"], " cfg2-reduced pre-activation")


def test_swiglu_pairing_closed_form(dev):
    """gate = even column, up = odd column: every output is 1.9296875 (swapped gives ~2.15)."""
    k, pairs = 64, 40
    dense = np.zeros((k, 2 * pairs), F32)
    dense[:, 0::2] = o.bf16_round(F32(0.02))
    dense[:, 1::2] = o.bf16_round(F32(0.03))
    w = o.quantize_frozen_weight(dense, group_size=k, scale_dtype="f32")
    case = {"m": 9, "k": k, "n": 2 * pairs, "x": np.ones((9, k), F32), "codes": w.codes, "scales": w.scales,
            "weight": w, "gamma": np.ones(k, F32), "swiglu": True}
    got, _ = wc.gpu_forward(case)
    assert np.all(got == F32(1.9296875))


@pytest.mark.parametrize("path", ["skinny", "tiled"])
def test_down_residual_decode_shape(dev, pkg, path):
    """Config 3: M16 K12288 N4096, 16 rank-32 adapters (one per row), residual; both kernels."""
    flags = pkg._native.FLAG_FORCE_SKINNY if path == "skinny" else pkg._native.FLAG_FORCE_TILED
    case = wc.make_case(16, 12288, 4096, n_adapters=16, rank=32, seed=7, residual=True, idx_mode="arange")
    st = wc.oracle_forward(case, return_stages=True)
    got, aux = wc.gpu_forward(case, flags=flags)
    _assert_integer_stages(aux, st)
    _assert_close(got, st["out"], f" cfg3 {path}")


@pytest.mark.parametrize("m,k,n,n_ad,rank,rms", [(1, 64, 17, 1, 8, False), (32, 2560, 6144, 4, 64, False),
                                                 (7, 1024, 520, 3, 24, True), (20, 4096, 2560, 0, 0, True),
                                                 (31, 384, 96, 2, 5, False)])
def test_skinny_path_shapes(dev, pkg, m, k, n, n_ad, rank, rms):
    """The split-K streaming kernel on ragged shapes, ranks and with the RMSNorm prologue."""
    case = wc.make_case(m, k, n, n_adapters=n_ad, rank=max(rank, 1), seed=m + k, rms=rms, residual=(m % 2 == 0))
    if n_ad:
        case["s"] = np.linspace(0.5, 2.0, n_ad).astype(F32)
    st = wc.oracle_forward(case, return_stages=True)
    got, aux = wc.gpu_forward(case, flags=pkg._native.FLAG_FORCE_SKINNY)
    if rms:
        np.testing.assert_array_equal(o.bf16_bits(aux["normalized"]), o.bf16_bits(st["normalized"]))
    _assert_integer_stages(aux, st)
    _assert_close(got, st["out"], f" skinny {m}x{k}x{n}")
    tiled, _ = wc.gpu_forward(case, flags=pkg._native.FLAG_FORCE_TILED)
    _assert_close(tiled, st["out"], f" tiled {m}x{k}x{n}")


@pytest.mark.parametrize("m,k,n,n_ad,rank,rms", [(33, 4096, 264, 3, 16, True), (47, 4096, 520, 2, 40, False),
                                                 (64, 4096, 1024, 0, 0, True), (96, 8192, 512, 5, 8, True),
                                                 (81, 12288, 776, 4, 64, False)])
def test_chunked_skinny_path(dev, pkg, m, k, n, n_ad, rank, rms):
    """Between 33 and 96 rows a call without SwiGLU over a long K whose weight fits the caches runs the streaming
    kernels on 32-row chunks: every stage against the oracle, ragged last chunks, and the tiled kernel on
    the same case (integer stages bit-equal between the two paths)."""
    nat = pkg._native
    assert nat.PATH_NAMES[nat.load().mi355_w8a8_forward_path(m, k, n, 0)] == "skinny-chunks"
    case = wc.make_case(m, k, n, n_adapters=n_ad, rank=max(rank, 1), seed=3 * m + k, rms=rms, residual=(m % 2 == 1))
    st = wc.oracle_forward(case, return_stages=True)
    got, aux = wc.gpu_forward(case)
    if rms:
        np.testing.assert_array_equal(o.bf16_bits(aux["normalized"]), o.bf16_bits(st["normalized"]))
    _assert_integer_stages(aux, st)
    _assert_close(got, st["out"], f" chunked {m}x{k}x{n}")
    tiled, aux_t = wc.gpu_forward(case, flags=pkg._native.FLAG_FORCE_TILED)
    _assert_close(tiled, st["out"], f" tiled {m}x{k}x{n}")
    for key in ("x_codes", "x_scales", "acc"):
        np.testing.assert_array_equal(aux[key], aux_t[key])


@pytest.mark.parametrize("m", [1, 64, 512])
@pytest.mark.parametrize("k,n", [(2560, 6144), (4096, 2560)])
def test_config4_student_t(dev, m, k, n):
    """Config 4: heavy-tailed activations, 4 adapters rank 64 alpha 128 (s = 2)."""
    case = wc.make_case(m, k, n, n_adapters=4, rank=64, alpha=128, seed=11 + m, student_t=True)
    st = wc.oracle_forward(case, return_stages=True)
    got, aux = wc.gpu_forward(case)
    _assert_integer_stages(aux, st)
    _assert_close(got, st["out"], f" cfg4 m{m} {k}x{n}")


def test_zero_inputs_finite(dev):
    case = wc.make_case(8, 64, 32, n_adapters=1, rank=8, seed=9, idx_mode="zero")
    case["x"][:] = 0
    got, aux = wc.gpu_forward(case)
    assert np.all(aux["x_codes"] == 0) and np.all(aux["x_scales"] == 1.0)
    assert np.all(got == 0) and np.all(np.isfinite(got))


def test_run_to_run_determinism(dev):
    case = wc.make_case(300, 512, 768, n_adapters=4, rank=16, seed=13, rms=True, swiglu=True)
    a = wc.gpu_forward(case, return_aux=False)
    b = wc.gpu_forward(case, return_aux=False)
    assert hashlib.sha256(a.tobytes()).hexdigest() == hashlib.sha256(b.tobytes()).hexdigest()


@pytest.mark.parametrize("shape", [
    dict(m=300, k=512, n=768, n_adapters=4, rank=16, rms=True, swiglu=True),
    dict(m=515, k=384, n=1000, n_adapters=5, rank=32),
    dict(m=100, k=448, n=520, n_adapters=3, rank=64, residual=True),
    dict(m=64, k=392, n=256, n_adapters=0),
    dict(m=700, k=2048, n=300, n_adapters=0, residual=True),
    dict(m=257, k=640, n=514, n_adapters=2, rank=8, swiglu=True),
    dict(m=513, k=1024, n=260, n_adapters=64, rank=16, idx_mode="arange"),
])
def test_tile_geometries_agree_bitwise(dev, pkg, shape):
    """The 256 x 128 geometry (32 x 32 x 32 MFMAs, two workgroups per CU) and the 256 x 256 geometry
    (16 x 16 x 64 MFMAs, one workgroup of eight waves per CU) agree: the int32 accumulators bit for bit, and so does the
    bf16 output wherever no LoRA term is added.  With LoRA the two low-rank products add their ranks in
    a different order inside the bf16 MFMAs (16 ranks per instruction against 32), which may move the
    last bit of an output: both stay inside the tolerance against the oracle and agree on >= 99.9 %."""
    shape = dict(shape)
    m, k, n = shape.pop("m"), shape.pop("k"), shape.pop("n")
    case = wc.make_case(m, k, n, seed=29, **shape)
    want = wc.oracle_forward(case, return_stages=True)
    narrow, aux_n = wc.gpu_forward(case, flags=pkg._native.FLAG_FORCE_TILED | pkg._native.FLAG_TILE_256X128)
    wide, aux_w = wc.gpu_forward(case, flags=pkg._native.FLAG_FORCE_TILED | pkg._native.FLAG_TILE_256X256)
    small, aux_s = wc.gpu_forward(case, flags=pkg._native.FLAG_FORCE_TILED | pkg._native.FLAG_TILE_128X128)
    pair, aux_p = wc.gpu_forward(case, flags=pkg._native.FLAG_FORCE_TILED | pkg._native.FLAG_TILE_256X128_PAIR)
    for aux in (aux_n, aux_w, aux_s, aux_p):
        assert np.array_equal(aux["acc"], want["acc"])
        assert np.array_equal(aux["x_codes"], want["x_codes"])
    # the 256 x 128 pair geometry is the 256 x 256 kernel with two waves side by side instead of four: the
    # same wave tile, the same operations per output
    assert np.array_equal(pair.view(np.uint32), wide.view(np.uint32))
    # the 128 x 128 geometry is the 256 x 128 kernel with one 32-row block per wave: the same operations per output
    assert np.array_equal(narrow.view(np.uint32), small.view(np.uint32))
    if shape.get("n_adapters", 1) == 0:
        assert np.array_equal(narrow.view(np.uint32), wide.view(np.uint32))
    else:
        assert np.mean(narrow.view(np.uint32) == wide.view(np.uint32)) >= 0.999
    _assert_close(narrow, want["out"], f" narrow {m}x{k}x{n}")
    _assert_close(wide, want["out"], f" wide {m}x{k}x{n}")


def test_tile_geometry_choice_and_contradictory_flags(dev, pkg):
    """Which geometry a call takes depends on its dimensions and flags only; asking for two is refused."""
    nat = pkg._native
    path = lambda m, k, n, flags=0: nat.PATH_NAMES.get(nat.load().mi355_w8a8_forward_path(m, k, n, flags))
    assert path(512, 2560, 6144) == "tiled-128x128"       # 4 x 48 tiles: all resident at once
    assert path(2048, 2560, 6144) == "tiled-256x256"      # 768 small tiles would queue; 192 wide ones fill the CUs
    assert path(4096, 4096, 24576) == "tiled-256x256"
    assert path(4096, 256, 4096) == "tiled-256x128"       # too few k steps for the 256 x 256 schedule
    assert path(16, 12288, 4096) == "skinny"
    assert path(64, 4096, 2560) == "skinny-chunks"
    assert path(128, 4096, 2560) == "tiled-128x128"
    assert path(96, 12288, 4096) == "skinny-chunks"
    assert path(128, 12288, 4096) == "tiled-128x128"
    assert path(64, 2560, 6144) == "tiled-128x128"
    assert path(512, 2560, 6144, nat.FLAG_TILE_256X128) == "tiled-256x128"
    assert path(4096, 4096, 24576, nat.FLAG_TILE_128X128) == "tiled-128x128"
    assert nat.load().mi355_w8a8_forward_path(512, 2560, 6144, nat.FLAG_TILE_256X128 | nat.FLAG_TILE_128X128) < 0
    # a forced geometry on a large call is still exact (1024 tiles of 128 x 128 on 512 workgroup slots)
    case = wc.make_case(1100, 512, 3000, n_adapters=3, rank=16, seed=41)
    want = wc.oracle_forward(case, return_stages=True)
    got, aux = wc.gpu_forward(case, flags=nat.FLAG_TILE_128X128)
    assert np.array_equal(aux["acc"], want["acc"])
    _assert_close(got, want["out"], " forced 128x128")


@pytest.mark.parametrize("seed", [1, 7])
def test_randomized_forward_sweep(dev, pkg, seed):
    """Sixty seeded draws over rows (1..1000), K, N, adapter counts (0..64, some without rows), ranks, RMSNorm,
    SwiGLU, residual and forced tile geometries: integer stages bit-equal to the oracle, outputs inside the
    tolerance.  Covers the path switches (decode kernels, 32-row chunks, the three tile geometries, adapters
    packed or on block boundaries) on shapes nobody picked by hand."""
    nat = pkg._native
    rng = np.random.default_rng(seed)
    for it in range(60):
        m = int(rng.choice([1, 5, 17, 33, 40, 64, 65, 96, 100, 129, 200, 257, 300, 511, 513, 640, 1000]))
        k = int(rng.choice([64, 136, 256, 392, 512, 768, 1024, 1536, 2048]))
        n = int(rng.choice([32, 96, 130, 256, 264, 520, 776, 1024, 1500]))
        n_ad = int(rng.choice([0, 1, 2, 3, 5, 8, 13, 32, 64]))
        rank = int(rng.choice([1, 3, 8, 16, 24, 32, 40, 64]))
        rms = bool(rng.integers(0, 2))
        swiglu = bool(rng.integers(0, 2)) and n % 2 == 0
        residual = (not swiglu) and bool(rng.integers(0, 2))
        idx_mode = str(rng.choice(["uniform", "arange", "zero"]))
        flags = int(rng.choice([0, 0, 0, nat.FLAG_FORCE_TILED, nat.FLAG_TILE_128X128,
                                nat.FLAG_FORCE_TILED | nat.FLAG_TILE_256X128, nat.FLAG_FORCE_TILED | nat.FLAG_TILE_256X256,
                                nat.FLAG_FORCE_TILED | nat.FLAG_TILE_256X128_PAIR]))
        if (flags & nat.FLAG_TILE_256X256) and k < 384:
            flags = nat.FLAG_FORCE_TILED
        what = f" m={m} k={k} n={n} adapters={n_ad} rank={rank} rms={rms} swiglu={swiglu} residual={residual} {idx_mode} flags={flags}"
        case = wc.make_case(m, k, n, n_adapters=n_ad, rank=rank, seed=1000 * seed + it, rms=rms, swiglu=swiglu,
                            residual=residual, idx_mode=idx_mode)
        if n_ad and idx_mode == "uniform" and rng.integers(0, 2):
            case["idx"] = (case["idx"] // 2 * 2 % n_ad).astype(np.int32)  # adapters without rows
        st = wc.oracle_forward(case, return_stages=True)
        got, aux = wc.gpu_forward(case, flags=flags)
        assert np.array_equal(aux["x_codes"], st["x_codes"]), what
        assert np.array_equal(aux["acc"], st["acc"]), what
        _assert_close(got, st["out"], what)
        if n_ad > 1:
            # A plan's first call lays out the LoRA operands and sorts the rows in that launch; its later
            # calls keep the operands and sort inside the quantizer (another order of the rows inside an
            # adapter's slots).  No output may depend on which of the two ran.
            import torch
            t = wc.to_torch(case, dev)
            plan = pkg.w8a8_lora.ForwardPlan(t["x"], t["weight"], t["a"], t["b"], t["s"], adapter_indices=t["idx"],
                                             rms_gamma=t.get("gamma"), eps=1e-6, residual=t.get("residual"),
                                             swiglu=swiglu, flags=flags)
            first = plan.run().clone()
            second = plan.run().clone()
            assert torch.equal(first, second), what
            np.testing.assert_array_equal(first.to(torch.float32).cpu().numpy(), got, err_msg=what)


def test_split2_flag_stays_in_tolerance(dev, pkg):
    case = wc.make_case(256, 512, 512, n_adapters=2, rank=32, seed=15)
    want = wc.oracle_forward(case)
    got = wc.gpu_forward(case, flags=pkg._native.FLAG_LORA_SPLIT2, return_aux=False)
    _assert_close(got, want, " split2")


def test_reference_call_surface(dev, pkg):
    """Opt-in and error conventions of skyrl/tx/kernels/rocm/w8a8_lora.py:57-59,844-849."""
    import torch

    w8 = pkg.w8a8_lora
    case = wc.make_case(4, 64, 32, n_adapters=1, rank=8, seed=17, idx_mode="zero")
    t = wc.to_torch(case, dev)
    with pytest.raises(RuntimeError, match="disabled by default"):
        w8.w8a8_lora_linear(t["x"], t["weight"], t["a"][0], t["b"][0], 1.0)
    with pytest.raises(TypeError, match="exact bool"):
        w8.w8a8_lora_linear(t["x"], t["weight"], t["a"][0], t["b"][0], 1.0, enabled=1)
    with pytest.raises(TypeError, match="BF16"):
        w8.w8a8_lora_linear(t["x"].float(), t["weight"], t["a"][0], t["b"][0], 1.0, enabled=True)
    with pytest.raises(ValueError):
        w8.w8a8_lora_linear(t["x"][:, :32], t["weight"], t["a"][0], t["b"][0], 1.0, enabled=True)
    with pytest.raises(ValueError):
        w8.w8a8_lora_linear(t["x"], t["weight"], t["a"][0][:, :4], t["b"][0], 1.0, enabled=True)
    with pytest.raises(ValueError):
        w8.w8a8_lora_linear(t["x"], t["weight"], t["a"][0], t["b"][0], 1.0, enabled=True, block_m=48)
    out = w8.w8a8_lora_linear(t["x"], t["weight"], t["a"][0], t["b"][0], 1.0, enabled=True)
    base = w8.w8a8_frozen_linear(t["x"], t["weight"], enabled=True)
    torch.cuda.synchronize()
    assert out.shape == (4, 32) and out.dtype == torch.bfloat16 and base.shape == (4, 32)
    want = o.quantized_lora_linear(case["x"], case["weight"], case["a"][0], case["b"][0], F32(1.0))
    assert o.within_tolerance(out.float().cpu().numpy(), want).all()
    # leading batch dimensions are flattened and restored
    x3 = t["x"].reshape(2, 2, 64)
    out3 = w8.w8a8_lora_linear(x3, t["weight"], t["a"][0], t["b"][0], 1.0, enabled=True)
    torch.cuda.synchronize()
    assert out3.shape == (2, 2, 32)
    assert torch.equal(out3.reshape(4, 32), out)


# ---------------------------------------------------------------------------------------
# grouped (per-expert) variant and the MoE composite
# ---------------------------------------------------------------------------------------
def _grouped_case(rng, sizes, k, n, rank, extra_rows=0):
    e = len(sizes)
    m = int(sum(sizes)) + extra_rows
    x = o.bf16_round(rng.standard_normal((m, k)).astype(F32))
    codes = rng.integers(-127, 128, (e, k, n), dtype=np.int8)
    scales = rng.uniform(0.001, 0.01, (e, n)).astype(F32)
    a = o.bf16_round((rng.standard_normal((e, k, rank)) * 0.02).astype(F32)) if rank else None
    b = o.bf16_round((rng.standard_normal((e, rank, n)) * 0.02).astype(F32)) if rank else None
    return m, x, codes, scales, a, b


@pytest.mark.parametrize("tile_rows", [64, 128])
@pytest.mark.parametrize("sizes,k,n,rank,swiglu,extra", [
    ([5, 0, 70, 33, 1, 64, 0, 129], 256, 512, 16, False, 0),
    ([40, 3, 0, 0, 200], 384, 1536, 16, True, 0),
    ([17, 90], 128, 96, 8, False, 9),
    ([64, 64, 64], 2048, 768, 0, False, 0),
    ([128, 300, 127, 129], 320, 1032, 32, True, 3),
])
def test_grouped_ragged_linear(dev, pkg, sizes, k, n, rank, swiglu, extra, tile_rows):
    import torch

    tile_flag = pkg._native.FLAG_GROUPED_TILE64 if tile_rows == 64 else pkg._native.FLAG_GROUPED_TILE128

    rng = np.random.default_rng(len(sizes) * 100 + k)
    m, x, codes, scales, a, b = _grouped_case(rng, sizes, k, n, rank, extra)
    s = F32(1.5)
    weights = [o.GroupQuantizedWeight(codes[e], scales[e:e + 1], k, k, 8, k) for e in range(len(sizes))]
    st = np.concatenate(([0], np.cumsum(sizes)))
    want_pre = np.zeros((m, n), F32)
    want_acc = np.zeros((m, n), np.int32)
    xc, xs = o.quantize_rows(x)
    for e, w in enumerate(weights):
        r0, r1 = int(st[e]), int(st[e + 1])
        if r1 > r0:
            if rank:
                want_pre[r0:r1] = o.quantized_lora_linear_f32(x[r0:r1], w, a[e], b[e], s)
            else:
                want_pre[r0:r1] = o.quantized_frozen_linear_f32(x[r0:r1], w)
            want_acc[r0:r1] = o.int_matmul(xc[r0:r1], codes[e])
    fused = o.bf16_round(want_pre)
    want = o.swiglu_from_interleaved(fused) if swiglu else fused
    w8 = pkg.w8a8_lora
    bf = lambda t: torch.from_numpy(np.ascontiguousarray(t)).to(dev).to(torch.bfloat16)
    gw = w8.prepare_grouped_weight(torch.from_numpy(codes).to(dev), torch.from_numpy(scales).to(dev))
    out, aux = w8.grouped_forward(bf(x), torch.tensor(sizes, dtype=torch.int32), gw,
                                  bf(a) if rank else None, bf(b) if rank else None, float(s) if rank else None,
                                  swiglu=swiglu, return_aux=True, flags=tile_flag)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    np.testing.assert_array_equal(aux["x_codes"].cpu().numpy(), xc)
    np.testing.assert_array_equal(aux["x_scales"].cpu().numpy().view(np.uint32), xs.view(np.uint32))
    np.testing.assert_array_equal(aux["acc"].cpu().numpy(), want_acc)
    assert np.all(got[int(st[-1]):] == 0)          # rows beyond the groups give zeros
    _assert_close(got, want, f" grouped {sizes} {k}x{n}")


def test_forward_under_inference_mode(dev, pkg):
    """Tensors made under ``torch.inference_mode()`` carry no version counter: the dense and the grouped plan
    and the group-scaled call take them all the same, pack the adapters on every run (a write to them could
    not be seen), and give the bits of the same calls on ordinary tensors."""
    import torch

    case = wc.make_case(70, 256, 192, n_adapters=3, rank=16, seed=5, rms=True)
    w8 = pkg.w8a8_lora

    def run(t):
        plan = w8.ForwardPlan(t["x"], t["weight"], t["a"], t["b"], t["s"], adapter_indices=t["idx"],
                              rms_gamma=t["gamma"], eps=1e-6)
        first = plan.run().clone()
        t["b"].mul_(-1.0)                 # no counter moves for an inference tensor: the next run must pack anyway
        second = plan.run().clone()
        sizes = torch.tensor([30, 0, 40], dtype=torch.int32, device=dev)
        gw = w8.prepare_grouped_weight(t["weight"].codes.unsqueeze(0).repeat(3, 1, 1).contiguous(),
                                       t["weight"].scales.reshape(1, -1).repeat(3, 1).contiguous())
        grouped = w8.grouped_forward(t["x"], sizes, gw, t["a"], t["b"], 1.0).clone()
        return first, second, grouped

    plain = run(wc.to_torch(case, dev))
    with torch.inference_mode():
        got = run(wc.to_torch(case, dev))
    for a, b in zip(plain, got):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    assert not torch.equal(plain[0].view(torch.int16), plain[1].view(torch.int16))


def test_grouped_plan_keeps_the_lora_packs_until_an_adapter_tensor_is_written(dev, pkg):
    """A grouped plan packs A and B on its first run, keeps the packs while neither tensor is written
    (the second run is told so and gives the same bits), and packs again after an in-place update."""
    import torch

    sizes, k, n, rank = [40, 3, 0, 70, 129], 384, 512, 16
    rng = np.random.default_rng(606)
    m, x, codes, scales, a, b = _grouped_case(rng, sizes, k, n, rank)
    s = F32(0.75)
    weights = [o.GroupQuantizedWeight(codes[e], scales[e:e + 1], k, k, 8, k) for e in range(len(sizes))]
    st = np.concatenate(([0], np.cumsum(sizes)))

    def oracle(bb):
        want = np.zeros((m, n), F32)
        for e, w in enumerate(weights):
            r0, r1 = int(st[e]), int(st[e + 1])
            if r1 > r0:
                want[r0:r1] = o.quantized_lora_linear_f32(x[r0:r1], w, a[e], bb[e], s)
        return o.bf16_round(want)

    w8 = pkg.w8a8_lora
    bf = lambda t: torch.from_numpy(np.ascontiguousarray(t)).to(dev).to(torch.bfloat16)
    gw = w8.prepare_grouped_weight(torch.from_numpy(codes).to(dev), torch.from_numpy(scales).to(dev))
    ta, tb = bf(a), bf(b)
    plan = w8.GroupedForwardPlan(bf(x), torch.tensor(sizes, dtype=torch.int32), gw, ta, tb, float(s))
    first = plan.run().clone()
    assert plan._packed_lora_key is not None
    second = plan.run().clone()           # packs kept
    assert torch.equal(first.view(torch.int16), second.view(torch.int16))
    _assert_close(first.float().cpu().numpy(), oracle(b), " grouped first run")
    tb.mul_(-1.0)                         # in place: the version counter moves, the next run packs again
    third = plan.run().clone()
    _assert_close(third.float().cpu().numpy(), oracle(-b), " grouped after new B")
    plan.keep_lora_pack = False
    fourth = plan.run().clone()
    assert torch.equal(third.view(torch.int16), fourth.view(torch.int16))


def test_moe_expert_mlp_reduced(dev, pkg):
    """Config 5 at reduced size: top-4 of 16 experts, hidden 256, intermediate 128, rank 16."""
    import torch

    rng = np.random.default_rng(55)
    t, h, inter, e, topk, r = 192, 256, 128, 16, 4, 16
    hidden = o.bf16_round(rng.standard_normal((t, h)).astype(F32))
    logits = rng.standard_normal((t, e)).astype(F32)
    gu_codes = rng.integers(-127, 128, (e, h, 2 * inter), dtype=np.int8)
    gu_scales = rng.uniform(0.001, 0.01, (e, 2 * inter)).astype(F32)
    dn_codes = rng.integers(-127, 128, (e, inter, h), dtype=np.int8)
    dn_scales = rng.uniform(0.001, 0.01, (e, h)).astype(F32)
    mk = lambda shape: o.bf16_round((rng.standard_normal(shape) * 0.02).astype(F32))
    gua, gub, da, db = mk((e, h, r)), mk((e, r, 2 * inter)), mk((e, inter, r)), mk((e, r, h))
    gu = [o.GroupQuantizedWeight(gu_codes[i], gu_scales[i:i + 1], h, h, 8, h) for i in range(e)]
    dn = [o.GroupQuantizedWeight(dn_codes[i], dn_scales[i:i + 1], inter, inter, 8, inter) for i in range(e)]
    want = o.moe_expert_mlp(hidden, logits, topk, gu, dn, gua, gub, da, db, F32(1.0))
    w8 = pkg.w8a8_lora
    bf = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev).to(torch.bfloat16)
    guw = w8.prepare_grouped_weight(torch.from_numpy(gu_codes).to(dev), torch.from_numpy(gu_scales).to(dev))
    dnw = w8.prepare_grouped_weight(torch.from_numpy(dn_codes).to(dev), torch.from_numpy(dn_scales).to(dev))
    got = w8.w8a8_moe_expert_mlp(bf(hidden), torch.from_numpy(logits).to(dev), topk, guw, dnw, bf(gua), bf(gub),
                                 bf(da), bf(db), 1.0, enabled=True)
    torch.cuda.synchronize()
    # Two quantized stages back to back: a one-ulp bf16 difference after the first stage changes a
    # row's absmax scale and so re-quantizes that whole row for the second stage.  The single
    # stages are held to the elementwise tolerance by the grouped tests above; the composite is
    # held to it for all but a vanishing fraction of elements.
    rep = wc.compare(got.float().cpu().numpy(), want)
    print(f"[parity] moe reduced {rep}", flush=True)
    assert rep["finite"] and rep["relative_l2"] < 1e-3 and rep["cosine"] >= 0.9999, rep
    assert rep["violations"] < 1e-3 * rep["size"], rep


def test_moe_expert_mlp_keeps_its_plans_between_calls(dev, pkg):
    """Without gradients the expert layer keeps its two grouped plans with the gate/up weight.  A second call
    (packs kept), a call with other hidden rows and logits (same buffers, another routing), a call after an
    adapter tensor was written in place (packs redone) and a call with another token count (new plans) all
    give what a layer with fresh weight objects -- so fresh plans -- gives, bit for bit."""
    import torch

    rng = np.random.default_rng(77)
    t, h, inter, e, topk, r = 96, 256, 128, 8, 2, 16
    gu_codes = torch.from_numpy(rng.integers(-127, 128, (e, h, 2 * inter), dtype=np.int8)).to(dev)
    gu_scales = torch.from_numpy(rng.uniform(0.001, 0.01, (e, 2 * inter)).astype(F32)).to(dev)
    dn_codes = torch.from_numpy(rng.integers(-127, 128, (e, inter, h), dtype=np.int8)).to(dev)
    dn_scales = torch.from_numpy(rng.uniform(0.001, 0.01, (e, h)).astype(F32)).to(dev)
    w8 = pkg.w8a8_lora
    bf = lambda shape, s=0.02: torch.from_numpy((rng.standard_normal(shape) * s).astype(F32)).to(dev).to(torch.bfloat16)
    lora = [bf((e, h, r)), bf((e, r, 2 * inter)), bf((e, inter, r)), bf((e, r, h))]
    guw, dnw = w8.prepare_grouped_weight(gu_codes, gu_scales), w8.prepare_grouped_weight(dn_codes, dn_scales)

    def kept(hidden, logits):
        return w8.w8a8_moe_expert_mlp(hidden, logits, topk, guw, dnw, *lora, 1.0, enabled=True).clone()

    def fresh(hidden, logits):
        a, b = w8.prepare_grouped_weight(gu_codes, gu_scales), w8.prepare_grouped_weight(dn_codes, dn_scales)
        return w8.w8a8_moe_expert_mlp(hidden, logits, topk, a, b, *[x.clone() for x in lora], 1.0, enabled=True).clone()

    same = lambda x, y: torch.equal(x.view(torch.int16), y.view(torch.int16))
    h1, l1 = bf((t, h), 1.0), torch.from_numpy(rng.standard_normal((t, e)).astype(F32)).to(dev)
    h2, l2 = bf((t, h), 1.0), torch.from_numpy(rng.standard_normal((t, e)).astype(F32)).to(dev)
    first, second = kept(h1, l1), kept(h1, l1)
    assert same(first, fresh(h1, l1)) and same(second, first)
    plan = w8._moe_inference_plans[guw]
    other = kept(h2, l2)
    assert w8._moe_inference_plans[guw] is plan and same(other, fresh(h2, l2)) and not same(other, first)
    lora[1].mul_(-1.0)                    # in place: the version counter moves, the next call packs again
    flipped = kept(h2, l2)
    assert w8._moe_inference_plans[guw] is plan and same(flipped, fresh(h2, l2)) and not same(flipped, other)
    h3, l3 = bf((40, h), 1.0), torch.from_numpy(rng.standard_normal((40, e)).astype(F32)).to(dev)
    fewer = kept(h3, l3)
    assert w8._moe_inference_plans[guw] is not plan and same(fewer, fresh(h3, l3))


@pytest.mark.parametrize("what", ["x_row", "x_elem", "w_col", "w_scale", "a_rank", "b_col", "scaling", "residual",
                                  "gamma", "index"])
def test_every_operand_matters(dev, what):
    """Operand sensitivity in the spirit of the reference's mutation list
    (rocm/probe_w8a8_lora_forward.py:1127-1190): changing any one operand changes the output, and
    the changed output still agrees with the oracle."""
    base = wc.make_case(40, 128, 96, n_adapters=3, rank=16, seed=41, rms=True, residual=True)
    got0 = wc.gpu_forward(base, return_aux=False)
    case = {k: (v.copy() if isinstance(v, np.ndarray) else v) for k, v in base.items()}
    if what == "x_row":
        case["x"][7] = o.bf16_round(case["x"][7] * F32(-1.5))
    elif what == "x_elem":
        case["x"][3, 17:18] = o.bf16_round(case["x"][3, 17:18] + F32(4.0))
    elif what == "w_col":
        case["codes"][:, 5] = -case["codes"][:, 5]
    elif what == "w_scale":
        case["scales"][0, 11] *= F32(2.0)
    elif what == "a_rank":
        case["a"][1, :, 15] = o.bf16_round(case["a"][1, :, 15] + F32(0.25))
    elif what == "b_col":
        case["b"][2, :, 95] = o.bf16_round(case["b"][2, :, 95] + F32(0.5))
    elif what == "scaling":
        case["s"][0] *= F32(3.0)
    elif what == "residual":
        case["residual"][39, 0:1] = o.bf16_round(case["residual"][39, 0:1] + F32(1.0))
    elif what == "gamma":
        case["gamma"][64] *= F32(1.5)
    elif what == "index":
        case["idx"][0] = (case["idx"][0] + 1) % 3
    case["weight"] = o.GroupQuantizedWeight(case["codes"], case["scales"], case["k"], case["k"], 8, case["k"])
    got1 = wc.gpu_forward(case, return_aux=False)
    assert np.any(got0 != got1), f"mutating {what} left the output unchanged"
    _assert_close(got1, wc.oracle_forward(case), f" mutated {what}")


def test_one_cast_after_the_f32_epilogue(dev):
    """The output is bf16(base_f32 + s * low_f32), not the sum of two early bf16 casts
    (skyrl/tx/kernels/quantized_lora.py:298-299, tests/tx/kernels/test_quantized_lora.py:178-199)."""
    case = wc.make_case(64, 256, 128, n_adapters=1, rank=16, seed=43, idx_mode="zero")
    got = wc.gpu_forward(case, return_aux=False)
    base = o.quantized_frozen_linear_f32(case["x"], case["weight"])
    low = (case["x"].astype(F32) @ case["a"][0].astype(F32)) @ case["b"][0].astype(F32)
    single = o.bf16_round(base + low * case["s"][0])
    early = o.bf16_round(o.bf16_round(base) + o.bf16_round(low * case["s"][0]))
    assert np.any(single != early)  # the inputs can tell the two apart
    differ = single != early
    agree_single = np.mean(o.bf16_bits(got)[differ] == o.bf16_bits(single)[differ])
    agree_early = np.mean(o.bf16_bits(got)[differ] == o.bf16_bits(early)[differ])
    assert agree_single > 0.95 and agree_early < 0.05, (agree_single, agree_early)


def test_quantizer_ties_round_to_even(dev, pkg):
    """Exact ties and near-ties of x / scale: rint is half-to-even on the correctly rounded
    quotient (skyrl/tx/kernels/quantized_lora.py:207-211)."""
    import torch

    k = 256
    rows = []
    half = (np.arange(k, dtype=F32) % 127) + F32(0.5)            # k + 0.5: exact ties when scale == 1
    half[0] = F32(127.0)                                         # absmax 127 -> scale exactly 1.0
    rows.append(half)
    rows.append(-half)
    third = (np.arange(k, dtype=F32) % 97) * F32(1.5)            # scale = 144/127: quotients near ties
    third[0] = F32(144.0)
    rows.append(third)
    tiny = ((np.arange(k, dtype=F32) % 63) - 31) * F32(2.0 ** -20)  # small magnitudes, scale far from 1
    rows.append(tiny)
    x = o.bf16_round(np.stack(rows))
    want_codes, want_scales = o.quantize_rows(x)
    case = wc.make_case(4, k, 64, n_adapters=0, seed=47)
    case["x"] = x
    for flags in (pkg._native.FLAG_FORCE_TILED, pkg._native.FLAG_FORCE_SKINNY):
        _, aux = wc.gpu_forward(case, flags=flags)
        np.testing.assert_array_equal(aux["x_codes"], want_codes)
        np.testing.assert_array_equal(aux["x_scales"].view(np.uint32), want_scales.reshape(-1).view(np.uint32))
    codes, scales = pkg.w8a8_lora.dynamic_quantize_rows(torch.from_numpy(x).to(dev).to(torch.bfloat16))
    np.testing.assert_array_equal(codes.cpu().numpy(), want_codes)


@pytest.mark.parametrize("m", [4, 80])
def test_largest_k(dev, m):
    """K = 16384 is the largest K the library accepts (both the decode and the tiled path)."""
    case = wc.make_case(m, 16384, 256, n_adapters=2, rank=8, seed=53, residual=True)
    st = wc.oracle_forward(case, return_stages=True)
    got, aux = wc.gpu_forward(case)
    _assert_integer_stages(aux, st)
    _assert_close(got, st["out"], f" K=16384 m={m}")


def test_same_named_fused_entry_points(dev, pkg):
    """``bf16_rms_gate_up_lora_swiglu_contiguous`` (delta RMSNorm weights) and ``bf16_lora_residual``
    in the reference's argument order on a quantized kernel; the residual form is differentiable with
    respect to x, A, B and the residual like the reference's custom VJP."""
    import torch

    gate_up = pkg.bf16_rms_gate_up_lora_swiglu_contiguous.bf16_rms_gate_up_lora_swiglu_contiguous
    down = pkg.bf16_lora_residual.bf16_lora_residual
    case = wc.make_case(48, 128, 96, n_adapters=1, rank=8, seed=31, rms=True, swiglu=True, idx_mode="zero")
    t = wc.to_torch(case, dev)
    delta = t["gamma"] - 1.0                                   # the reference stores the delta
    out = gate_up(t["x"], delta, t["weight"], t["a"][0], t["b"][0], 1.0, enabled=True, eps=1e-6)
    torch.cuda.synchronize()
    case_delta = dict(case, gamma=(F32(1.0) + (case["gamma"] - F32(1.0)).astype(F32)).astype(F32))
    assert wc.compare(out.float().cpu().numpy(), wc.oracle_forward(case_delta))["violations"] == 0

    case = wc.make_case(40, 128, 64, n_adapters=1, rank=8, seed=32, residual=True, idx_mode="zero")
    t = wc.to_torch(case, dev)
    x = t["x"].clone().requires_grad_(True)
    a = t["a"][0].clone().requires_grad_(True)
    b = t["b"][0].clone().requires_grad_(True)
    res = t["residual"].clone().requires_grad_(True)
    out = down(x, t["weight"], a, b, 1.0, res, enabled=True)
    assert wc.compare(out.detach().float().cpu().numpy(), wc.oracle_forward(case))["violations"] == 0
    cot = o.bf16_round(np.random.default_rng(5).standard_normal((40, 64)).astype(F32))
    (out.float() * torch.from_numpy(cot).to(dev)).sum().backward()
    torch.cuda.synchronize()
    want = o.quantized_lora_linear_bwd(case["x"], case["weight"], case["a"][0], case["b"][0], F32(1.0), cot,
                                       relaxed_weight=True)
    for got, ref in ((x.grad, want[0]), (a.grad, want[1]), (b.grad, want[2])):
        assert wc.compare(got.float().cpu().numpy(), ref)["violations"] == 0
    np.testing.assert_array_equal(res.grad.float().cpu().numpy(), cot)     # the residual's cotangent is dy


@pytest.mark.parametrize("token_tile_size", [1, 4, 6, 16])
def test_bounded_frozen_lora_linear_forward_equation_across_token_tiles(dev, pkg, token_tile_size):
    """``bounded_frozen_lora_linear`` (skyrl/tx/kernels/bounded_lora.py:121-140, :245-255) on a quantized
    kernel: ``x @ W8A8 + s * (x @ A) @ B + residual`` for x of shape [2, 5, K] with the rank-8 single adapter,
    scaling 0.375 and residual of the reference's own test
    (tests/tx/kernels/test_bounded_lora.py:23-43).  The result is the oracle's, does not depend on
    ``token_tile_size``, and is what the same rows give when they are passed in pieces of that size."""
    import torch

    bounded = pkg.bounded_lora.bounded_frozen_lora_linear
    case = wc.make_case(10, 16, 7, n_adapters=1, rank=8, seed=33, residual=True, idx_mode="zero")
    case["s"] = np.asarray([0.375], F32)
    t = wc.to_torch(case, dev)
    x3, res3 = t["x"].reshape(2, 5, 16), t["residual"].reshape(2, 5, 7)
    out = bounded(x3, t["weight"], t["a"][0], t["b"][0], 0.375, residual=res3, token_tile_size=token_tile_size)
    ref_tile = bounded(x3, t["weight"], t["a"][0], t["b"][0], 0.375, residual=res3, token_tile_size=512)
    torch.cuda.synchronize()
    assert tuple(out.shape) == (2, 5, 7)
    assert torch.equal(out.view(torch.int16), ref_tile.view(torch.int16))
    assert wc.compare(out.float().cpu().numpy().reshape(10, 7), wc.oracle_forward(case))["violations"] == 0
    # (a piece is copied out: the C ABI wants 16-byte-aligned pointers, and a 7-column row is 14 bytes)
    pieces = [bounded(t["x"][r0:r0 + token_tile_size].clone(), t["weight"], t["a"][0], t["b"][0], 0.375,
                      residual=t["residual"][r0:r0 + token_tile_size].clone(), token_tile_size=token_tile_size)
              for r0 in range(0, 10, token_tile_size)]
    torch.cuda.synchronize()
    assert torch.equal(torch.cat(pieces).view(torch.int16), out.reshape(10, 7).view(torch.int16))


def test_lora_pack_is_reused_until_the_adapters_change(dev, pkg):
    """A plan keeps the transposed A / packed B in its workspace while the adapter tensors are unchanged
    (the second run is told so and must give the same bits), and packs again after an in-place update."""
    import torch

    w8 = pkg.w8a8_lora
    case = wc.make_case(600, 512, 768, n_adapters=3, rank=16, seed=51, rms=True, swiglu=True)
    t = wc.to_torch(case, dev)
    plan = w8.ForwardPlan(t["x"], t["weight"], t["a"], t["b"], t["s"], adapter_indices=t["idx"],
                          rms_gamma=t["gamma"], eps=1e-6, swiglu=True)
    first = plan.run().clone()
    assert plan._packed_lora_key is not None
    second = plan.run().clone()          # FLAG_LORA_PACK_VALID
    assert torch.equal(first.view(torch.int16), second.view(torch.int16))
    _assert_close(first.to(torch.float32).cpu().numpy(), wc.oracle_forward(case), " first run")
    # an in-place update of B bumps its version: the next run packs again and follows the new values
    t["b"].mul_(2.0)
    third = plan.run().clone()
    case2 = dict(case, b=case["b"] * np.float32(2.0))
    _assert_close(third.to(torch.float32).cpu().numpy(), wc.oracle_forward(case2), " after the update")
    assert not torch.equal(third.view(torch.int16), first.view(torch.int16))


def test_lora_pack_survives_another_row_count_and_geometry(dev, pkg):
    """The packed LoRA operands sit at the start of the workspace at places that depend on
    (k, n, n_adapters, rank) only: a call with another m, other adapter indices and another tile geometry
    on the same workspace may keep them (MI355_W8A8_FLAG_LORA_PACK_VALID) and gives the bits of a call
    that packs for itself."""
    import torch

    w8, nat = pkg.w8a8_lora, pkg._native
    big = wc.make_case(700, 512, 768, n_adapters=3, rank=16, seed=52, residual=True)
    tb = wc.to_torch(big, dev)
    plan_big = w8.ForwardPlan(tb["x"], tb["weight"], tb["a"], tb["b"], tb["s"], adapter_indices=tb["idx"],
                              residual=tb["residual"], flags=nat.FLAG_TILE_256X128)
    plan_big.run()  # packs A and B into its workspace
    small = dict(big)
    rng = np.random.default_rng(5)
    rows = rng.permutation(700)[:150]
    small.update(m=150, x=big["x"][rows], residual=big["residual"][rows],
                 idx=rng.integers(0, 3, 150).astype(np.int32))
    ts = wc.to_torch(small, dev)
    ts["a"], ts["b"], ts["s"], ts["weight"] = tb["a"], tb["b"], tb["s"], tb["weight"]
    plan_small = w8.ForwardPlan(ts["x"], ts["weight"], ts["a"], ts["b"], ts["s"], adapter_indices=ts["idx"],
                                residual=ts["residual"], flags=nat.FLAG_TILE_128X128)
    own = plan_small.run().clone()  # packs into its own workspace
    # the same call on the larger call's workspace, told to keep what is there
    plan_small.problem.workspace = plan_big.problem.workspace
    plan_small.problem.workspace_bytes = plan_big.problem.workspace_bytes
    plan_small.keep_lora_pack = False
    kept = plan_small.run(nat.FLAG_LORA_PACK_VALID).clone()
    torch.cuda.synchronize()
    assert torch.equal(own.view(torch.int16), kept.view(torch.int16))
    _assert_close(kept.to(torch.float32).cpu().numpy(), wc.oracle_forward(small), " kept pack, other m")


@pytest.mark.parametrize("m", [8192, 8200])
def test_routing_inside_and_outside_the_quantizer_launch(dev, m):
    """Up to 8192 rows the quantizer's workgroups sort the adapter indices themselves; beyond, a workgroup
    of the preparation launch does.  Both sides of the switch, with an empty adapter and out-of-range
    indices (clamped like an XLA gather), against the oracle."""
    case = wc.make_case(m, 256, 512, n_adapters=5, rank=8, seed=61)
    idx = case["idx"].copy()
    idx[idx == 3] = 1          # adapter 3 has no rows
    idx[5], idx[77] = -4, 99   # clamped to 0 and 4
    case["idx"] = idx
    want = wc.oracle_forward(dict(case, idx=np.clip(idx, 0, 4)), return_stages=True)
    got, aux = wc.gpu_forward(case, flags=0)
    _assert_integer_stages(aux, want)
    _assert_close(got, want["out"], f" routing m={m}")


def test_decode_regrouped_b_is_reused_until_b_or_the_indices_change(dev, pkg):
    """The decode kernels keep B regrouped per row in the workspace; a plan reuses it while B and the
    adapter indices are unchanged and rebuilds it after either is written."""
    import torch

    w8 = pkg.w8a8_lora
    case = wc.make_case(12, 1024, 768, n_adapters=5, rank=16, seed=71, residual=True)
    t = wc.to_torch(case, dev)
    plan = w8.ForwardPlan(t["x"], t["weight"], t["a"], t["b"], t["s"], adapter_indices=t["idx"], residual=t["residual"])
    first = plan.run().clone()
    second = plan.run().clone()          # regrouped B kept
    assert torch.equal(first.view(torch.int16), second.view(torch.int16))
    _assert_close(first.to(torch.float32).cpu().numpy(), wc.oracle_forward(case), " decode first run")
    new_idx = (case["idx"] + 2) % 5
    plan.adapter_indices.copy_(torch.from_numpy(new_idx.astype(np.int32)).to(dev))
    third = plan.run().clone()
    _assert_close(third.to(torch.float32).cpu().numpy(), wc.oracle_forward(dict(case, idx=new_idx.astype(np.int32))),
                  " decode after new indices")
    t["b"].mul_(-1.0)
    fourth = plan.run().clone()
    _assert_close(fourth.to(torch.float32).cpu().numpy(),
                  wc.oracle_forward(dict(case, idx=new_idx.astype(np.int32), b=-case["b"])), " decode after new B")
