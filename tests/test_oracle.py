"""Pins the CPU oracle against what the reference's own files fix: its LUT
literal and bit-trick constants, its reshape/permute layout code, its test
parameters (group lists, all-ones x), and library routines (torch float8 decode,
torch bf16 multiply, torch fp64 matmul).  No GPU needed."""
import numpy as np
import pytest
import torch

import oracle
from oracle import layouts as L


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def from_bits(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


# ---------------------------------------------------------------- e2m1 / e4m3
def test_e2m1_matches_reference_lut_literal():
    # test_group_gemm_fp4.py:6-8 (magnitudes) and :22 (sign = bit 3)
    levels = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    for code in range(16):
        v = oracle.e2m1_decode(code)
        assert v == (-1.0 if code & 8 else 1.0) * levels[code & 7]
    assert np.signbit(np.float32(oracle.e2m1_decode(8)))  # code 8 is -0.0


def test_e2m1_matches_python_bit_trick():
    # fp4_dequant, test_group_gemm_fp4.py:97-102: ((w&8)<<12)|((w&7)<<6) as bf16, times 0x7E80
    w = torch.arange(16, dtype=torch.int16)
    bits = ((w & 0x0008) << 12) | ((w & 0x0007) << 6)
    mul = torch.tensor([0x7E80], dtype=torch.int16).view(torch.bfloat16)
    val = (bits.view(torch.bfloat16) * mul).float()
    for code in range(16):
        assert val[code].item() == oracle.e2m1_decode(code)
        assert bool(torch.signbit(val[code])) == bool(code & 8)


def test_e2m1_matches_kernel_bit_trick():
    # preCastFP4Weight, grouped_gemm/op_kernel/antiquant_impl.h:41-85:
    # sign-extended nibble << 9, & 0x8E00, reinterpret fp16, times 0x7400 (2^14)
    for code in range(16):
        s = code - 16 if code & 8 else code
        bits = np.array([(s << 9) & 0x8E00], dtype=np.uint16)
        v = bits.view(np.float16).astype(np.float32) * np.array([0x7400], dtype=np.uint16).view(np.float16).astype(np.float32)
        assert v[0] == np.float32(oracle.e2m1_decode(code))


def test_e4m3_matches_torch_float8_and_nan_codes():
    codes = torch.arange(256, dtype=torch.uint8)
    ref = codes.view(torch.float8_e4m3fn).float()
    for c in range(256):
        v = oracle.e4m3_decode(c)
        if c & 0x7F == 0x7F:
            assert v == (-480.0 if c & 0x80 else 480.0)  # no NaN handling in the reference
        else:
            assert v == ref[c].item(), c


def test_e4m3_matches_python_bit_trick():
    # anti_quant_fp8, test_group_gemm_fp8.py:11-14
    w = torch.arange(256, dtype=torch.int16)
    bits = ((w & 0x0080) << 8) | ((w & 0x007F) << 4)
    mul = torch.tensor([0x7B80], dtype=torch.int16).view(torch.bfloat16)
    val = (bits.view(torch.bfloat16) * mul).float()
    for c in range(256):
        assert val[c].item() == oracle.e4m3_decode(c)


def test_bf16_rounding_matches_torch():
    rng = np.random.default_rng(0)
    f = rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-20, 20, 20000).astype(np.float32)
    f = np.concatenate([f, np.array([0.0, -0.0, 1.00390625, 1.01171875, 3.3895314e38, np.inf, -np.inf], np.float32)])
    got = oracle.f32_to_bf16_bits(f)
    ref = bf16_bits(torch.from_numpy(f).to(torch.bfloat16))
    assert np.array_equal(got, ref)
    for v in f[:200]:
        assert oracle.lib().orc_f32_to_bf16(float(v)) == int(oracle.f32_to_bf16_bits(np.array([v]))[0])


# ------------------------------------------------------------- fp4 pre-shuffle
def test_preshuffle_closed_form_matches_reshape_permute():
    rng = np.random.default_rng(1)
    G, K, N = 2, 128, 512
    codes = rng.integers(0, 16, (G, K, N), dtype=np.uint8)
    ckpt = L.pack_nibbles_last(np.ascontiguousarray(codes.transpose(0, 2, 1)))   # [G, N, K/2]
    cont = L.fp4ref_from_checkpoint(ckpt).view(np.uint8)                          # [G, K, N/2]
    flat = cont.reshape(G, -1)
    for g in range(G):
        for k in range(K):
            for n in range(0, N, 7):
                idx, nib = oracle.fp4ref_locate(k, n, N)
                byte = int(flat[g, idx])
                assert ((byte >> 4) if nib else (byte & 15)) == codes[g, k, n]


def test_preshuffle_brute_force_tiny_and_roundtrip():
    # one tile, every byte tagged with its own source index: brute-force scan
    K, NB = 64, 128
    src = np.arange(K * NB, dtype=np.int32).reshape(1, K, NB)
    t = src.reshape(1, 4, 2, 8, 1, 8, 4, 4).transpose(0, 2, 1, 5, 4, 6, 3, 7).reshape(K * NB)
    for k in range(K):
        for c in range(NB):
            idx, _ = oracle.fp4ref_locate(k, 2 * c, 2 * NB)
            assert t[idx] == k * NB + c
    rng = np.random.default_rng(2)
    w = rng.integers(-128, 128, (3, 192, 256), dtype=np.int8)
    assert np.array_equal(L.fp4ref_stage2_inverse(L.fp4ref_stage2(w)), w)
    assert sorted(L.fp4ref_stage2(w).reshape(-1).tolist()) == sorted(w.reshape(-1).tolist())


def test_stage1_matches_reference_int16_form():
    # repack_weight, test_group_gemm_fp4.py:105-117, done literally with torch int16 views
    rng = np.random.default_rng(3)
    ckpt = rng.integers(0, 256, (2, 64, 32), dtype=np.uint8)       # [G, N, K/2]
    tw = torch.from_numpy(ckpt).to(torch.int16)
    tw = ((tw & 0x00F0) << 4) | (tw & 0x000F)
    nw = tw.view(torch.uint8).reshape(2, 64, 64).transpose(-2, -1).contiguous().view(torch.int16)
    nw = (((nw & 0x0F00) >> 4) | (nw & 0x000F)).to(torch.int8)
    assert np.array_equal(L.fp4ref_stage1(ckpt), nw.numpy())


# -------------------------------------------------------------------- dequant
def test_dequant_fp4_matches_torch_bf16_multiply():
    # twin of fp4_dequant + the per-block loop, test_group_gemm_fp4.py:97-102, :205-207
    g = torch.Generator().manual_seed(4)
    R, C, B = 64, 256, 32
    codes = torch.randint(0, 16, (R, C), generator=g, dtype=torch.uint8)
    scale = (torch.rand(R, C // B, generator=g) * (2**-2 - 2**-8) + 2**-8).to(torch.bfloat16)
    packed = L.pack_nibbles_last(codes.numpy())
    got = oracle.dequant_fp4_bf16(packed, bf16_bits(scale), B)
    w16 = codes.to(torch.int16)
    bits = ((w16 & 8) << 12) | ((w16 & 7) << 6)
    w = bits.view(torch.bfloat16) * torch.tensor([0x7E80], dtype=torch.int16).view(torch.bfloat16)
    for i in range(C // B):
        w[:, i * B:(i + 1) * B] *= scale[:, i].unsqueeze(-1)
    assert np.array_equal(got, bf16_bits(w))
    # code 8 with any positive scale must give -0.0 (0x8000)
    z = oracle.dequant_fp4_bf16(np.full((1, 16), 0x88, np.uint8), bf16_bits(torch.ones(1, 1, dtype=torch.bfloat16)), 32)
    assert (z == 0x8000).all()


# --------------------------------------------------------------- expand_weight
def _mk_fp4ref(rng, G, K, N):
    codes = rng.integers(0, 16, (G, K, N), dtype=np.uint8)
    ckpt = L.pack_nibbles_last(np.ascontiguousarray(codes.transpose(0, 2, 1)))
    w = L.fp4ref_from_checkpoint(ckpt)
    scale = torch.from_numpy(rng.uniform(0.01, 0.5, (G, K // 16, N)).astype(np.float32)).to(torch.bfloat16)
    return codes, w, scale


def test_expand_fp4ref_against_lut_and_torch_multiply():
    rng = np.random.default_rng(5)
    G, K, N = 2, 128, 256
    codes, w, scale = _mk_fp4ref(rng, G, K, N)
    lut = torch.tensor([0, .5, 1, 1.5, 2, 3, 4, 6, -0., -.5, -1, -1.5, -2, -3, -4, -6], dtype=torch.bfloat16)
    for g in range(G):
        dec = lut[torch.from_numpy(codes[g].astype(np.int64))]
        s = scale[g].repeat_interleave(16, dim=0)
        ref_bf16 = (dec * s).float().numpy()                 # bf16*bf16 -> one RNE
        ref_f32 = (dec.float() * s.float()).numpy()
        assert np.array_equal(oracle.expand_weight(oracle.FMT_FP4_REF, w, bf16_bits(scale), None, g, True), ref_bf16)
        assert np.array_equal(oracle.expand_weight(oracle.FMT_FP4_REF, w, bf16_bits(scale), None, g, False), ref_f32)


def test_expand_fp8ref_against_reference_reshape_form():
    rng = np.random.default_rng(6)
    G, K, N = 2, 256, 384
    w = rng.integers(0, 256, (G, K, N), dtype=np.uint8)
    scale = rng.standard_normal((G, K // 128, N // 128)).astype(np.float32)
    for rb in (True, False):
        ref = L.fp8ref_dequant_numpy(w, scale, rb)
        for g in range(G):
            assert np.array_equal(oracle.expand_weight(oracle.FMT_FP8_REF, w, scale, None, g, rb), ref[g])


def test_expand_int8_int4_fp4b32_bf16_closed_forms():
    rng = np.random.default_rng(7)
    G, K, N = 2, 256, 64
    # int8: (q + off) * scale, two fp32 roundings then RNE to bf16
    q = rng.integers(-127, 128, (G, K, N), dtype=np.int8)
    sc = torch.from_numpy(rng.uniform(1e-3, 1e-2, (G, N)).astype(np.float32)).to(torch.bfloat16)
    of = torch.from_numpy(rng.uniform(-2, 2, (G, N)).astype(np.float32)).to(torch.bfloat16)
    for g in range(G):
        ref = ((torch.from_numpy(q[g]).float() + of[g].float()) * sc[g].float())
        got = oracle.expand_weight(oracle.FMT_INT8, q, bf16_bits(sc), bf16_bits(of), g, True)
        assert np.array_equal(got, ref.to(torch.bfloat16).float().numpy())
    # int4: (q - 8) * scale[k // gs, n]
    c4 = rng.integers(0, 16, (G, K, N), dtype=np.uint8)
    w4 = L.pack_nibbles_last(c4)
    s4 = torch.from_numpy(rng.uniform(1e-3, 1e-2, (G, K // 128, N)).astype(np.float32)).to(torch.bfloat16)
    for g in range(G):
        ref = (torch.from_numpy(c4[g].astype(np.float32)) - 8.0) * s4[g].float().repeat_interleave(128, dim=0)
        got = oracle.expand_weight(oracle.FMT_INT4, w4, bf16_bits(s4), None, g, True)
        assert np.array_equal(got, ref.to(torch.bfloat16).float().numpy())
    # fp4_b32: K-contiguous container [G, N, K/2], scale [G, N, K/32]; equals the
    # stand-alone dequant of the [G*N, K/2] matrix, transposed
    cb = rng.integers(0, 16, (G, N, K), dtype=np.uint8)
    wb = L.pack_nibbles_last(cb)
    sb = torch.from_numpy(rng.uniform(2**-8, 2**-2, (G, N, K // 32)).astype(np.float32)).to(torch.bfloat16)
    dq = oracle.dequant_fp4_bf16(wb.reshape(G * N, K // 2), bf16_bits(sb).reshape(G * N, K // 32), 32)
    dq = oracle.bf16_bits_to_f32(dq).reshape(G, N, K)
    for g in range(G):
        got = oracle.expand_weight(oracle.FMT_FP4_B32, wb, bf16_bits(sb), None, g, True)
        assert np.array_equal(got, dq[g].T)
    # fp4_b16: the same container with one scale per 16 k (the checkpoint orientation of
    # test_group_gemm_fp4.py:46-64); equals the reference test's own dequant expression
    # (do_dequant_b, :67-75: decode * b_s per block of 16) and the stand-alone block-16 dequant
    s16 = torch.from_numpy(rng.uniform(2**-8, 2**-2, (G, N, K // 16)).astype(np.float32)).to(torch.bfloat16)
    dq = oracle.dequant_fp4_bf16(wb.reshape(G * N, K // 2), bf16_bits(s16).reshape(G * N, K // 16), 16)
    dq = oracle.bf16_bits_to_f32(dq).reshape(G, N, K)
    lut = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])
    cbt = torch.from_numpy(cb.astype(np.int64))
    vals = torch.where((cbt >> 3).bool(), -1.0, 1.0) * lut[cbt & 7]
    ref16 = (vals.view(G, N, K // 16, 16) * s16.float().view(G, N, K // 16, 1)).view(G, N, K)
    for g in range(G):
        got = oracle.expand_weight(oracle.FMT_FP4_B16, wb, bf16_bits(s16), None, g, True)
        assert np.array_equal(got, dq[g].T)
        assert np.array_equal(got, ref16[g].to(torch.bfloat16).float().numpy().T)
        got = oracle.expand_weight(oracle.FMT_FP4_B16, wb, bf16_bits(s16), None, g, False)
        assert np.array_equal(got, ref16[g].numpy().T)
    # bf16 [G, N, K]
    wf = torch.randn(G, N, K, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    got = oracle.expand_weight(oracle.FMT_BF16, bf16_bits(wf), None, None, 1, True)
    assert np.array_equal(got, wf[1].float().numpy().T)


def test_scale_merge_and_transpose_against_torch_in_place_multiply():
    """anti_quant_fp8_scale (test_group_gemm_fp4.py:86-94) multiplies the bf16 scale tensor in
    place by the fp32 second-level scale; torch computes that product in fp32 and rounds to
    nearest even.  Then the test transposes to [G, K/16, N] (:185-186)."""
    rng = np.random.default_rng(11)
    G, N, KB = 3, 8, 12
    sc = torch.from_numpy(rng.uniform(1.0, 448.0, (G, N, KB)).astype(np.float32)).to(torch.bfloat16)
    # one factor per expert (scale_2.shape[-2] == 1)
    s2 = torch.from_numpy(rng.uniform(1e-4, 1e-2, (G, 1, 1)).astype(np.float32))
    ref = sc.clone()
    ref *= s2
    ref = ref.to(torch.bfloat16).transpose(1, 2).contiguous()
    got = L.fp4ref_scale_from_checkpoint(bf16_bits(sc), s2.numpy().reshape(G, 1))
    assert np.array_equal(got, bf16_bits(ref))
    # two factors: first / second half of the N rows
    s2 = torch.from_numpy(rng.uniform(1e-4, 1e-2, (G, 2, 1)).astype(np.float32))
    ref = sc.clone()
    ref[..., : N // 2, :] *= s2[..., 0, :].unsqueeze(-1)
    ref[..., N // 2 :, :] *= s2[..., 1, :].unsqueeze(-1)
    ref = ref.to(torch.bfloat16).transpose(1, 2).contiguous()
    got = L.fp4ref_scale_from_checkpoint(bf16_bits(sc), s2.numpy().reshape(G, 2))
    assert np.array_equal(got, bf16_bits(ref))
    # no second-level scale: a plain transpose
    assert np.array_equal(L.fp4ref_scale_from_checkpoint(bf16_bits(sc)), bf16_bits(sc.transpose(1, 2).contiguous()))


def test_routing_sort_brute_force_and_invariants():
    """route_sort is a stable sort of the (token, choice) pairs by expert id: checked against a
    pure-Python insertion into per-expert lists, and against what any such sort must satisfy."""
    from oracle import routing as R

    rng = np.random.default_rng(21)
    T, k, E = 37, 3, 7
    ids = rng.integers(0, E, (T, k)).astype(np.int32)
    ids[5, 1] = -1      # dropped
    ids[9, 0] = E       # dropped
    gl, row_token, roc = R.route_sort(ids, E)
    buckets = [[] for _ in range(E)]
    for t in range(T):
        for j in range(k):
            if 0 <= ids[t, j] < E:
                buckets[ids[t, j]].append((t, j))
    flat = [tj for b in buckets for tj in b]
    assert list(gl) == list(np.cumsum([len(b) for b in buckets]))
    assert [t for t, _ in flat] == list(row_token)
    for r, (t, j) in enumerate(flat):
        assert roc[t * k + j] == r
    assert roc[5 * k + 1] == -1 and roc[9 * k + 0] == -1
    # invariants: expert ids of the sorted rows are non-decreasing, row_of_choice is a bijection onto the rows
    valid = roc >= 0
    sorted_ids = np.empty(valid.sum(), dtype=np.int64)
    sorted_ids[roc[valid]] = ids.reshape(-1)[valid]
    assert (np.diff(sorted_ids) >= 0).all() and gl[-1] == valid.sum()
    assert sorted(roc[valid]) == list(range(valid.sum()))


def test_routing_topk_against_torch_topk_and_softmax():
    from oracle import routing as R

    g = torch.Generator().manual_seed(4)
    logits = torch.randn(50, 64, generator=g)
    ids, w = R.route_topk(logits.numpy(), 8)
    tv, ti = torch.topk(logits, 8, dim=1)          # distinct values: no tie-breaking involved
    assert np.array_equal(ids, ti.numpy().astype(np.int32))
    assert np.allclose(w, torch.softmax(logits, dim=1).gather(1, ti).numpy(), rtol=1e-6, atol=1e-8)
    # ties go to the lower expert id
    tie = np.zeros((1, 6), dtype=np.float32)
    tie[0, 4] = 1.0
    ids, _ = R.route_topk(tie, 3)
    assert list(ids[0]) == [4, 0, 1]


def test_swiglu_interleaved_against_torch_silu_and_explicit_columns():
    rng = np.random.default_rng(31)
    z = (rng.standard_normal((5, 16)) * 3).astype(np.float32)
    got = oracle.bf16_bits_to_f32(oracle.swiglu_interleaved(z))
    zt = torch.from_numpy(z).double()
    gate = torch.stack([zt[:, 0::4], zt[:, 1::4]], dim=2).reshape(5, 8)     # gate 2j, 2j+1 of every group of 4
    up = torch.stack([zt[:, 2::4], zt[:, 3::4]], dim=2).reshape(5, 8)
    ref = (torch.nn.functional.silu(gate) * up).float().to(torch.bfloat16).float().numpy()
    assert np.array_equal(got, ref)
    # one group by hand: columns (g0, g1, u0, u1) = (1, -2, 3, 4)
    one = oracle.bf16_bits_to_f32(oracle.swiglu_interleaved(np.array([[1.0, -2.0, 3.0, 4.0]], dtype=np.float32)))
    assert np.allclose(one, [[1.0 / (1.0 + np.exp(-1.0)) * 3.0, -2.0 / (1.0 + np.exp(2.0)) * 4.0]], rtol=2 ** -8)


def test_swiglu_blocked16_against_torch_silu():
    rng = np.random.default_rng(32)
    z = (rng.standard_normal((3, 64)) * 3).astype(np.float32)
    got = oracle.bf16_bits_to_f32(oracle.swiglu_blocked16(z))
    zt = torch.from_numpy(z).double()
    gate = torch.cat([zt[:, 0:16], zt[:, 32:48]], dim=1)     # first 16 columns of every block of 32
    up = torch.cat([zt[:, 16:32], zt[:, 48:64]], dim=1)
    ref = (torch.nn.functional.silu(gate) * up).float().to(torch.bfloat16).float().numpy()
    assert np.array_equal(got, ref)


# ---------------------------------------------------------------- grouped_gemm
@pytest.mark.parametrize("group_list", [[2, 3, 4, 256], [12, 25, 44, 48], [1, 2, 3, 4], [0, 0, 5, 5], [3, 3, 3, 3]])
def test_grouped_gemm_against_torch_fp64(group_list):
    # group lists of the reference tests (test_group_gemm_fp4.py:172, _fp8.py:50, gemv :172) + empty experts
    rng = np.random.default_rng(8)
    G, K, N = 4, 128, 256
    M = max(group_list[-1], 1) + 3        # trailing rows stay untouched
    codes, w, scale = _mk_fp4ref(rng, G, K, N)
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16)
    y16, y32 = oracle.grouped_gemm(oracle.FMT_FP4_REF, bf16_bits(x), w, bf16_bits(scale), None, group_list, want_f32=True)
    ref = torch.zeros(M, N, dtype=torch.float64)
    prev = 0
    for g, end in enumerate(group_list):
        Wg = torch.from_numpy(oracle.expand_weight(oracle.FMT_FP4_REF, w, bf16_bits(scale), None, g, True)).double()
        ref[prev:end] = x[prev:end].double() @ Wg
        prev = end
    assert np.allclose(y32, ref.numpy(), rtol=1e-5, atol=1e-4)
    assert (y16[group_list[-1]:] == 0).all() and (y32[group_list[-1]:] == 0).all()
    assert np.array_equal(y16, oracle.f32_to_bf16_bits(y32))
    # row mask: only the listed rows are produced
    mask = np.zeros(M, np.uint8)
    mask[::3] = 1
    ym = oracle.grouped_gemm(oracle.FMT_FP4_REF, bf16_bits(x), w, bf16_bits(scale), None, group_list, row_mask=mask)
    assert np.array_equal(ym[mask == 1], y16[mask == 1]) and (ym[mask == 0] == 0).all()


def test_grouped_gemm_fp8_all_ones_x_is_column_sums():
    # reference fp8 tests use x = ones: y[m, n] = sum_k W_g[k, n] (test_group_gemm_fp8.py:49-50)
    rng = np.random.default_rng(9)
    G, M, K, N = 4, 48, 256, 384
    w = rng.integers(0, 255, (G, K, N), dtype=np.uint8)
    scale = rng.standard_normal((G, 2, 3)).astype(np.float32)
    gl = [12, 25, 44, 48]
    x = torch.ones(M, K, dtype=torch.bfloat16)
    _, y32 = oracle.grouped_gemm(oracle.FMT_FP8_REF, bf16_bits(x), w, scale, None, gl, want_f32=True)
    Wd = L.fp8ref_dequant_numpy(w, scale, True).astype(np.float64)
    prev = 0
    for g, end in enumerate(gl):
        col = Wd[g].sum(0)
        assert np.allclose(y32[prev:end], np.broadcast_to(col, (end - prev, N)), rtol=1e-5, atol=1e-2)
        prev = end


def test_grouped_gemm_rejects_bad_group_list():
    rng = np.random.default_rng(10)
    codes, w, scale = _mk_fp4ref(rng, 2, 64, 256)
    x = np.zeros((4, 64), np.uint16)
    with pytest.raises(RuntimeError):
        oracle.grouped_gemm(oracle.FMT_FP4_REF, x, w, bf16_bits(scale), None, [3, 2])
    with pytest.raises(RuntimeError):
        oracle.grouped_gemm(oracle.FMT_FP4_REF, x, w, bf16_bits(scale), None, [2, 9])


def test_oracle_under_address_and_ub_sanitizers():
    """`make -C oracle asan`: every entry point of the C oracle on exactly sized heap buffers under
    AddressSanitizer and UBSan (host code only; the GPU side has no sanitizer on this pool)."""
    import os
    import subprocess

    here = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle")
    r = subprocess.run(["make", "-C", here, "-B", "asan"], capture_output=True, text=True, timeout=300)
    out = r.stdout + r.stderr
    if "ASan runtime does not come first" in out:
        pytest.skip("another preloaded library keeps AddressSanitizer from starting in this environment")
    assert r.returncode == 0, out[-2000:]
    assert "sanitize_check ok" in out


def test_int8_one_fma_equals_the_two_rounded_operations_where_the_kernel_uses_it():
    """The int8 decode of the GPU kernel replaces (q + offset) * scale, two rounded fp32 operations, by one fma
    q * scale + offset * scale where the sum cannot round: offset 0 or |offset| in [2^-8, 2^22], scale in
    [2^-60, 2^60].  Checked here on every q against random bf16 offsets and scales of that domain, bit for bit;
    the fma is evaluated exactly in float64 (16-bit products at most 2^30 apart) and rounded once."""
    rng = np.random.default_rng(77)
    n = 20000
    def bf16_of(mag_lo, mag_hi, signed):
        e = rng.integers(mag_lo, mag_hi, n)                     # exponent
        m = rng.integers(128, 256, n).astype(np.float64) / 128  # 8-bit significand in [1, 2)
        v = np.ldexp(m, e)
        if signed:
            v *= rng.choice([-1.0, 1.0], n)
        return v.astype(np.float32)
    off = bf16_of(-8, 22, True)
    off[: n // 10] = 0.0
    off[n // 10: n // 10 + 50] = np.float32(2.0 ** -8)
    off[n // 10 + 50: n // 10 + 100] = np.float32(255.0 / 128 * 2.0 ** 21)   # largest allowed bf16 below 2^22
    scale = bf16_of(-60, 60, False)
    assert (oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(off)) == off).all()
    assert (oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(scale)) == scale).all()
    for q in range(-128, 128):
        qf = np.float32(q)
        two = (qf + off) * scale                                             # float32 add, float32 multiply
        one = (np.float64(q) * scale.astype(np.float64) + off.astype(np.float64) * scale.astype(np.float64)).astype(np.float32)
        assert np.array_equal(two.view(np.uint32), one.view(np.uint32)), q
