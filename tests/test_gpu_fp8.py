"""GPU parity of the fp8 (OCP e4m3fn) pieces: the quantising element-wise
kernels against the oracle's scalar conversion (bit-exact where the input is
exactly representable work, neighbouring-code acceptance where f32 libm
differences can move a value across a rounding boundary), the fp8 MFMA mmt4d on
N(0,1) inputs against f64 accumulation, and the MLP block end to end.

The reference has no fp8 mmt4d (its type enum ends at 0x0A,
runtime/src/iree/builtins/ukernel/exported_bits.h:29-41); what pins these tests
is the e4m3 decode/encode pair, which the CPU suite checks against the known
answers of runtime/src/iree/base/internal/math_test.cc:420-475, and the fact
that a product of two e4m3 values is exact in f32."""
import numpy as np
import pytest

import gpucase
import ukref
from iree_amd import flags as F
from iree_amd import synth

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-2, 1e-3
TABLE = ukref.f8e4m3_decode_table().astype(np.float64)
_FINITE = np.array([v for v in range(256) if np.isfinite(TABLE[v])], dtype=np.uint8)
_ORDER = _FINITE[np.argsort(TABLE[_FINITE], kind="stable")]
_SORTED = TABLE[_ORDER]


def encode_e4m3(values):
    """float array -> e4m3fn codes through the oracle's scalar encoder (OCP
    rounding, saturating)."""
    enc = ukref.oracle().oracle_f32_to_f8e4m3
    flat = np.asarray(values, dtype=np.float32).reshape(-1)
    return np.array([enc(float(v), 1, 1) for v in flat], dtype=np.uint8).reshape(np.shape(values))


def quantize_np(values):
    """Nearest-even e4m3 code of each value (vectorised, for large arrays);
    checked against the scalar oracle encoder in test_vectorised_encoder."""
    v = np.clip(np.asarray(values, dtype=np.float64), -448.0, 448.0)
    # The e4m3 grid: spacing 2^(e-3) for |v| in [2^e, 2^(e+1)), 2^-9 below 2^-6.
    mag = np.abs(v)
    e = np.floor(np.log2(np.maximum(mag, 2.0 ** -6)))
    e = np.clip(e, -6, 8)
    ulp = 2.0 ** (e - 3)
    q = np.rint(mag / ulp) * ulp          # rint = round half to even
    q = np.minimum(q, 448.0)
    idx = np.searchsorted(_SORTED, np.where(v < 0, -q, q))
    idx = np.clip(idx, 0, _SORTED.size - 1)
    codes = _ORDER[idx]
    # searchsorted lands on -0.0/+0.0 ambiguously; fix the sign of zeros
    zero = q == 0
    codes = np.where(zero, np.where(np.signbit(v), 0x80, 0x00), codes).astype(np.uint8)
    return codes


def test_vectorised_encoder_matches_the_oracle_encoder():
    rng = np.random.default_rng(0)
    vals = np.concatenate([rng.standard_normal(4000) * s for s in (1e-3, 0.05, 1.0, 30.0, 300.0)])
    vals = np.concatenate([vals, TABLE[_FINITE], [0.0, -0.0, 464.0, 500.0, -1e9, 2.0 ** -10, 3 * 2.0 ** -10]])
    vals = vals.astype(np.float32)
    assert np.array_equal(quantize_np(vals), encode_e4m3(vals))


def test_quantize_f16_all_bit_patterns(uk, cuda):
    """Every f16 bit pattern, three scales: bit-exact against
    f32(f16) * inv_scale -> oracle e4m3 encoder (RNE, saturating, NaN kept)."""
    import torch
    bits = np.arange(65536, dtype=np.uint16)
    src = torch.from_numpy(bits.view(np.int16)).cuda()
    for inv_scale in (1.0, 0.37, 3.0, 448.0 / 5.5):
        out = torch.zeros(65536, dtype=torch.uint8, device="cuda")
        uk.quantize_f16_to_f8e4m3(src, out, 65536, inv_scale)
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        with np.errstate(invalid="ignore"):
            x = bits.view(np.float16).astype(np.float32) * np.float32(inv_scale)
        nan = np.isnan(x)
        want = quantize_np(np.where(nan, 0, x))
        assert np.array_equal(got[~nan], want[~nan]), inv_scale
        assert np.all((got[nan] & 0x7F) == 0x7F)
    # spot check of the vectorised expectation against the scalar oracle
    sample = bits[::97].view(np.float16).astype(np.float32)
    sample = sample[np.isfinite(sample)]
    assert np.array_equal(quantize_np(sample), encode_e4m3(sample))


def test_quantize_ragged_and_unaligned(uk, cuda):
    import torch
    x = synth.normal_f16(5, 1003, 40.0)
    for off in (0, 1, 3):
        n = 1003 - off
        src = torch.from_numpy(x.view(np.int16)).cuda()
        out = torch.full((1003 + 8,), 0xAA, dtype=torch.uint8, device="cuda")
        uk.quantize_f16_to_f8e4m3(src[off:], out[off:], n, 0.5)
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        want = quantize_np(x[off:].astype(np.float32) * np.float32(0.5))
        assert np.array_equal(got[off:off + n], want)
        assert np.all(got[:off] == 0xAA) and np.all(got[off + n:] == 0xAA)


@pytest.mark.parametrize("rows,cols,ld,loose", [(64, 256, 256, False), (45, 48, 56, True), (1, 16, 16, False),
                                                (33, 2064, 2064, False), (2048, 4096, 4096, False)])
def test_quantize_pack_in_one_pass(uk, cuda, rows, cols, ld, loose):
    """The fused quantisation + pack: bit-exact against the oracle encoder laid
    out by the pack oracle's rule (tile (i, j) row r = matrix row 32 i + r,
    columns 16 j .. 16 j + 16, rows past the end zero), and equal to the two
    separate entry points; all f16 bit patterns occur in the first case; memory
    between outer rows of a loose tiled buffer stays untouched."""
    import torch
    if rows * cols >= 65536:
        x = np.resize(np.arange(65536, dtype=np.uint16), rows * ld)
        x = np.where((x & 0x7C00) == 0x7C00, x & 0x83FF, x).astype(np.uint16)     # no Inf / NaN here
    else:
        x = synth.normal_f16(rows + cols, rows * ld, 30.0).view(np.uint16)
    inv_scale = 0.37
    M1, K1 = -(-rows // 32), cols // 16
    stride = cols * 32 + (64 if loose else 0)
    src = torch.from_numpy(x.view(np.int16)).cuda()
    out = torch.full((M1 * stride,), 0xAA, dtype=torch.uint8, device="cuda")
    uk.quantize_pack_f8e4m3(src, out, rows, cols, inv_scale, ld=ld, out_stride0=stride)
    q = torch.zeros(rows * ld, dtype=torch.uint8, device="cuda")
    uk.quantize_f16_to_f8e4m3(src, q, rows * ld, inv_scale)
    two = torch.full((M1 * stride,), 0xAA, dtype=torch.uint8, device="cuda")
    uk.pack(q, two, rows, cols, M1, K1, 32, 16, 0, F.PACK_TYPE_I8I8, in_stride0=ld, out_stride0=stride)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.array_equal(got, two.cpu().numpy())
    xm = x.view(np.float16).reshape(rows, ld)[:, :cols].astype(np.float32) * np.float32(inv_scale)
    want = np.zeros((M1 * 32, cols), np.uint8)
    want[:rows] = quantize_np(xm.reshape(-1)).reshape(rows, cols)
    want = want.reshape(M1, 32, K1, 16).transpose(0, 2, 1, 3).reshape(M1, cols * 32)
    g = got.reshape(M1, stride)
    assert np.array_equal(g[:, :cols * 32], want)
    assert np.all(g[:, cols * 32:] == 0xAA)
    with pytest.raises(uk.UkError):
        uk.quantize_pack_f8e4m3(src, out, rows, cols - 3, inv_scale, ld=ld, out_stride0=stride)


def _acceptable_codes(v64):
    """Codes an implementation accurate to 1e-5 relative may produce."""
    lo = quantize_np(v64 * (1 - 1e-5) - 1e-12)
    hi = quantize_np(v64 * (1 + 1e-5) + 1e-12)
    return lo, hi


def _silu_expect(g, u, gs, us, os):
    g64 = g.astype(np.float64) * gs
    u64 = u.astype(np.float64) * us
    silu = np.array([ukref.oracle().oracle_silu_mul(float(a), float(b)) for a, b in zip(g64.reshape(-1)[:64], u64.reshape(-1)[:64])])
    v = g64 / (1.0 + np.exp(-g64)) * u64
    assert np.allclose(v.reshape(-1)[:64], silu, rtol=1e-14, atol=0)   # numpy form == the oracle's libm form
    return v * os


def _check_codes(got, v64, v_lo=None, v_hi=None):
    """`got` must lie between the codes of the ends of the interval the exact
    value may fall in: [v_lo, v_hi] if given, else v64 (1 +- 1e-5)."""
    if v_lo is None:
        lo, hi = _acceptable_codes(v64)
    else:
        lo, hi = quantize_np(v_lo), quantize_np(v_hi)
    a, b = TABLE[lo], TABLE[hi]
    g = TABLE[got]
    ok = (g >= np.minimum(a, b)) & (g <= np.maximum(a, b))
    assert np.all(ok), (int((~ok).sum()), v64[~ok][:4], got[~ok][:4])
    # and almost all agree with the exact rounding
    assert np.mean(got == quantize_np(v64)) > 0.99


@pytest.mark.parametrize("rows,cols,ld", [(64, 256, 512), (5, 37, 41), (33, 128, 128)])
def test_silu_mul_quantize_row_major(uk, cuda, rows, cols, ld):
    import torch
    rng = np.random.default_rng(rows * cols)
    buf = (rng.standard_normal((rows, 2 * ld)) * 6).astype(np.float32)
    gs, us, os = 0.7, 1.3, 2.5
    dev = torch.from_numpy(buf.reshape(-1)).cuda()
    out = torch.zeros(rows * cols, dtype=torch.uint8, device="cuda")
    # gate = left half of each row, up = right half (one fused [rows][2 ld] result)
    uk.silu_mul_quantize(dev, dev[ld:], out, rows, cols, 2 * ld, gs, us, os)
    torch.cuda.synchronize()
    got = out.cpu().numpy().reshape(rows, cols)
    want = _silu_expect(buf[:, :cols], buf[:, ld:ld + cols], gs, us, os)
    _check_codes(got, want)


def test_silu_mul_quantize_tiled_equals_row_major_on_unpacked_tiles(uk, cuda):
    import torch
    M1, N1 = 3, 5
    rng = np.random.default_rng(7)
    # tiled f32 result with 2 N1 + 1 outer columns (one spare) : gate at 1.., up at 1 + N1..
    cols1 = 2 * N1 + 1
    acc = (rng.standard_normal((M1, cols1, 32, 32)) * 5).astype(np.float32)
    gs, us, os = 0.9, 1.1, 3.0
    out = torch.full((M1 * N1 * 1024 + 64,), 0xEE, dtype=torch.uint8, device="cuda")
    uk.silu_mul_quantize_tiled(torch.from_numpy(acc.reshape(-1)).cuda(), cols1 * 1024, 1, 1 + N1,
                               out, N1 * 1024, M1, N1, gs, us, os)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.all(got[M1 * N1 * 1024:] == 0xEE)
    got = got[:M1 * N1 * 1024].reshape(M1, 2 * N1, 32, 16)          # LHS tiles 32x16
    gate = acc[:, 1:1 + N1].transpose(0, 2, 1, 3).reshape(M1 * 32, N1 * 32)
    up = acc[:, 1 + N1:1 + 2 * N1].transpose(0, 2, 1, 3).reshape(M1 * 32, N1 * 32)
    got_rm = got.transpose(0, 2, 1, 3).reshape(M1 * 32, N1 * 32)
    _check_codes(got_rm, _silu_expect(gate, up, gs, us, os))
    # identical bits to the row-major kernel on the unpacked operands
    rm = torch.zeros(M1 * 32 * N1 * 32, dtype=torch.uint8, device="cuda")
    uk.silu_mul_quantize(torch.from_numpy(np.ascontiguousarray(gate).reshape(-1)).cuda(),
                         torch.from_numpy(np.ascontiguousarray(up).reshape(-1)).cuda(), rm,
                         M1 * 32, N1 * 32, N1 * 32, gs, us, os)
    torch.cuda.synchronize()
    assert np.array_equal(rm.cpu().numpy().reshape(M1 * 32, N1 * 32), got_rm)


def test_scale_f32(uk, cuda):
    import torch
    x = synth.normal_f32(3, 1027)
    for off in (0, 1):
        t = torch.from_numpy(x.copy()).cuda()
        uk.scale_f32(t[off:], 1027 - off, 0.3)
        torch.cuda.synchronize()
        want = x.copy()
        want[off:] *= np.float32(0.3)
        assert np.array_equal(t.cpu().numpy(), want)


def test_fp8_mmt4d_normal_inputs_within_tolerance(uk, cuda):
    """e4m3 x e4m3 -> f32 on quantised N(0,1) inputs, K = 2048, +-accumulate,
    against f64 accumulation of the same codes."""
    rng = np.random.default_rng(11)
    M, N, K0 = 5, 6, 16
    K = 2048 // K0

    def gen(rng, tf, which, n):
        if which == 2:
            return rng.standard_normal(n).astype(np.float32)
        return quantize_np(rng.standard_normal(n) * (0.5 if which else 1.0))

    for acc in (False, True):
        case = ukref.Mmt4dCase(rng, F.MMT4D_TYPE_F8E4M3F8E4M3F32, M, N, K, 32, 32, K0,
                               accumulate=acc, generator=gen)
        assert uk.mmt4d_info(32, 32, K0, F.MMT4D_TYPE_F8E4M3F8E4M3F32) == 1
        got = case.written_region(gpucase.run_mmt4d(case))
        want = case.written_region(case.run_oracle(f64=True))
        assert np.all(np.abs(got - want) <= ATOL + RTOL * np.abs(want))
        # far tighter in practice (fp8 MFMA accumulation error, see the MLP test)
        assert np.max(np.abs(got - want)) < 2e-3


def test_fp8_mlp_block_small(uk, cuda):
    """The whole block at hidden 256, ffn 512, 64 tokens. The intermediate h is
    checked code by code against the f64 formula evaluated on the GPU's own
    gate/up accumulators' exact counterparts, and the output against f64
    accumulation over the GPU's h codes (identical quantised operands)."""
    import torch
    M, H, Fn = 64, 256, 512
    x = synth.normal_f16(1, M * H).reshape(M, H)
    wg = synth.normal_f32(2, Fn * H, 0.02).reshape(Fn, H)
    wu = synth.normal_f32(3, Fn * H, 0.02).reshape(Fn, H)
    wd = synth.normal_f32(4, H * Fn, 0.02).reshape(H, Fn)
    sg, su, sd = (float(np.abs(w).max()) / 448.0 for w in (wg, wu, wd))
    sx = float(np.abs(x.astype(np.float32)).max()) / 448.0
    wg_q, wu_q, wd_q = quantize_np(wg / sg), quantize_np(wu / su), quantize_np(wd / sd)
    xq = quantize_np(x.astype(np.float32) * np.float32(1.0 / sx))
    g = (TABLE[xq] @ TABLE[wg_q].T) * (sx * sg)
    u = (TABLE[xq] @ TABLE[wu_q].T) * (sx * su)
    h = g / (1.0 + np.exp(-g)) * u
    sh = float(np.abs(h).max()) / 448.0

    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a).reshape(-1)).cuda()  # noqa: E731
    mlp = uk.Fp8Mlp(H, Fn, dev(wg_q), dev(wu_q), dev(wd_q), sg, su, sd, sx, sh, max_tokens=M,
                    fused=False)
    y = torch.zeros(M * H, dtype=torch.float32, device="cuda")
    mlp(dev(x.view(np.int16)), y, M)
    # the fused gate/up + SiLU kernel: same accumulators, same arithmetic, same bits
    fused = uk.Fp8Mlp(H, Fn, dev(wg_q), dev(wu_q), dev(wd_q), sg, su, sd, sx, sh, max_tokens=M)
    y2 = torch.full((M * H,), 7.0, dtype=torch.float32, device="cuda")
    fused(dev(x.view(np.int16)), y2, M)
    torch.cuda.synchronize()
    assert np.array_equal(fused.x_tiles.cpu().numpy(), mlp.x_tiles.cpu().numpy())   # one-pass quantise + pack
    assert np.array_equal(fused.h_tiles.cpu().numpy(), mlp.h_tiles.cpu().numpy())
    assert np.array_equal(y2.cpu().numpy(), y.cpu().numpy())
    # x codes: bit-exact
    assert np.array_equal(mlp.xq.cpu().numpy().reshape(M, H), xq)
    # h codes (as LHS tiles 32x16 -> row-major)
    hq = mlp.h_tiles.cpu().numpy().reshape(M // 32, Fn // 16, 32, 16).transpose(0, 2, 1, 3).reshape(M, Fn)
    # The kernel starts from the gate/up values the fp8 MFMA accumulated. That
    # instruction sums its 64 products with less than f32 precision: measured
    # on MI355X, one instruction is off by up to 2e-5 of the sum of the
    # magnitudes of its terms (the error of longer sums grows slower than the
    # sum). Accept the codes of every h reachable inside a box of twice that
    # (plus 1e-5 relative for the f32 exp and divide).
    eg = 4e-5 * (np.abs(TABLE[xq]) @ np.abs(TABLE[wg_q]).T) * (sx * sg)
    eu = 4e-5 * (np.abs(TABLE[xq]) @ np.abs(TABLE[wu_q]).T) * (sx * su)
    silu = lambda t: t / (1.0 + np.exp(-t))  # noqa: E731
    corners = np.stack([silu(g + a * eg) * (u + b * eu) for a in (-1, 1) for b in (-1, 1)]) / sh
    lo, hi = corners.min(axis=0), corners.max(axis=0)
    pad = 1e-5 * np.maximum(np.abs(lo), np.abs(hi)) + 1e-12
    _check_codes(hq, h / sh, lo - pad, hi + pad)
    want = (TABLE[hq] @ TABLE[wd_q].T) * (sh * sd)
    got = y.cpu().numpy().reshape(M, H).astype(np.float64)
    assert np.all(np.abs(got - want) <= ATOL + RTOL * np.abs(want))
    assert np.max(np.abs(got - want)) <= 1e-4 * np.abs(want).max()


@pytest.mark.parametrize("type_flag,K0", [(F.MMT4D_TYPE_F8E4M3F8E4M3F32, 16), (F.MMT4D_TYPE_F16F16F32, 8)])
@pytest.mark.parametrize("M1,P,K1", [(1, 1, 4), (3, 5, 7), (9, 33, 12), (64, 64, 5)])
def test_fused_gate_up_silu_matches_unfused(uk, cuda, type_flag, K0, M1, P, K1):
    """mmt4d_silu_mul_f8e4m3 on interleaved gate/up tiles against plain mmt4d
    followed by silu_mul_quantize_tiled on the de-interleaved accumulators:
    identical bytes (ragged macro tiles, partial last K step, every tile variant
    the launcher picks at these sizes), loose output pitch respected."""
    import torch
    rng = np.random.default_rng(M1 * 100 + P + K1)
    n_l, n_r = M1 * K1 * 32 * K0, 2 * P * K1 * 32 * K0
    if type_flag == F.MMT4D_TYPE_F16F16F32:
        lhs = (rng.standard_normal(n_l) * 0.5).astype(np.float16).view(np.uint16)
        rhs = (rng.standard_normal(n_r) * 0.5).astype(np.float16).view(np.uint16)
    else:
        lhs, rhs = quantize_np(rng.standard_normal(n_l)), quantize_np(rng.standard_normal(n_r))
    dl, dr = torch.from_numpy(lhs.view(np.uint8)).cuda(), torch.from_numpy(rhs.view(np.uint8)).cuda()
    gs, us, os_ = 0.8, 1.2, 0.7
    pitch = P * 1024 + 64
    fused = torch.full((M1 * pitch,), 0xEE, dtype=torch.uint8, device="cuda")
    uk.mmt4d_silu_mul_f8e4m3(dl, dr, fused, M1, 2 * P, K1, K0, type_flag, gs, us, os_, out_stride0=pitch)
    acc = torch.zeros(M1 * 2 * P * 1024, dtype=torch.float32, device="cuda")
    uk.mmt4d(dl, dr, acc, M1, 2 * P, K1, 32, 32, K0, type_flag)
    a4 = acc.view(M1, P, 2, 1024)
    split = torch.cat([a4[:, :, 0], a4[:, :, 1]], dim=1).contiguous()     # [M1][gate tiles | up tiles]
    want = torch.zeros(M1 * P * 1024, dtype=torch.uint8, device="cuda")
    uk.silu_mul_quantize_tiled(split, 2 * P * 1024, 0, P, want, P * 1024, M1, P, gs, us, os_)
    torch.cuda.synchronize()
    got = fused.cpu().numpy().reshape(M1, pitch)
    assert np.array_equal(got[:, :P * 1024].reshape(-1), want.cpu().numpy())
    assert np.all(got[:, P * 1024:] == 0xEE)


def test_fused_gate_up_silu_invalid_arguments(uk, cuda):
    import torch
    t = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    mm = F.MMT4D_TYPE_F8E4M3F8E4M3F32
    with pytest.raises(uk.UkError) as e:
        uk.mmt4d_silu_mul_f8e4m3(t, t, t, 1, 3, 4, 16, mm, 1.0, 1.0, 1.0)        # odd N
    assert e.value.status == F.STATUS_INVALID_ARGUMENT
    with pytest.raises(uk.UkError):
        uk.mmt4d_silu_mul_f8e4m3(t, t, t, 1, 2, 4, 16, mm | F.MMT4D_ACCUMULATE, 1.0, 1.0, 1.0)
    with pytest.raises(uk.UkError) as e:
        uk.mmt4d_silu_mul_f8e4m3(t, t, t, 1, 2, 4, 16, F.MMT4D_TYPE_S8S8S32, 1.0, 1.0, 1.0)
    assert e.value.status == F.STATUS_UNIMPLEMENTED
    with pytest.raises(uk.UkError) as e:
        uk.mmt4d_silu_mul_f8e4m3(t[1:], t, t, 1, 2, 4, 16, mm, 1.0, 1.0, 1.0)    # misaligned operand
    assert e.value.status == F.STATUS_UNIMPLEMENTED
    uk.mmt4d_silu_mul_f8e4m3(t, t, t, 0, 2, 4, 16, mm, 1.0, 1.0, 1.0)             # M == 0: nothing to do


def test_fp8_mlp_block_full_size_sampled_tokens(uk, cuda):
    """The block at its real size (2048 tokens, hidden 4096, ffn 14336): for a
    sample of token rows, h codes against the f64 formula on the same quantised
    operands (within the fp8 MFMA's accumulation error), and y against f64
    accumulation over the GPU's own h codes: |err| <= 1e-3 + 1e-2 |y|."""
    import torch
    M, H, Fn = 2048, 4096, 14336
    # Operands from the seeded integer-only generators (activations N(0, 1),
    # weights N(0, 0.02)), so that the host side can regenerate the same bytes
    # on any machine. A weight matrix is 8 M generated elements repeated, each
    # repetition rotated by another 977 elements (58.7 M elements per matrix
    # from the generator itself would take the host a minute).
    x = torch.from_numpy(synth.normal_f16(990, M * H)).cuda()
    codes, scales = [], []
    piece = 1 << 23
    for wi, n_el in enumerate((Fn * H, Fn * H, H * Fn)):
        base = torch.from_numpy(synth.normal_f16(991 + wi, piece, 0.02)).cuda()
        w = torch.empty(n_el, dtype=torch.float16, device="cuda")
        for k, first in enumerate(range(0, n_el, piece)):
            n = min(piece, n_el - first)
            w[first:first + n] = torch.roll(base, 977 * k)[:n]
        del base
        sc = float(w.float().abs().max()) / 448.0
        q = torch.empty(n_el, dtype=torch.uint8, device="cuda")
        uk.quantize_f16_to_f8e4m3(w, q, n_el, 1.0 / sc)
        codes.append(q)
        scales.append(sc)
        del w
    sg, su, sd = scales
    sx = float(x.float().abs().max()) / 448.0
    rows = np.array([0, 1, 31, 32, 777, 1024, 2047])
    # reference gate/up for the sampled rows -> the scale of h
    xq = quantize_np(x.cpu().numpy().astype(np.float32).reshape(M, H)[rows] * np.float32(1.0 / sx))
    wg = TABLE[codes[0].cpu().numpy().reshape(Fn, H)]
    wu = TABLE[codes[1].cpu().numpy().reshape(Fn, H)]
    X = TABLE[xq]
    gt = (X @ wg.T) * (sx * sg)
    ut = (X @ wu.T) * (sx * su)
    h = gt / (1.0 + np.exp(-gt)) * ut
    sh = float(np.abs(h).max()) * 1.5 / 448.0          # head room for the rows not sampled
    mlp = uk.Fp8Mlp(H, Fn, codes[0], codes[1], codes[2], sg, su, sd, sx, sh, max_tokens=M)
    y = torch.zeros(M * H, dtype=torch.float32, device="cuda")
    mlp(x, y, M)
    torch.cuda.synchronize()
    xt = mlp.x_tiles.cpu().numpy().reshape(M // 32, H // 16, 32, 16).transpose(0, 2, 1, 3).reshape(M, H)
    assert np.array_equal(xt[rows], xq)
    hq = mlp.h_tiles.cpu().numpy().reshape(M // 32, Fn // 16, 32, 16).transpose(0, 2, 1, 3).reshape(M, Fn)[rows]
    eg = 4e-5 * (np.abs(X) @ np.abs(wg).T) * (sx * sg)
    eu = 4e-5 * (np.abs(X) @ np.abs(wu).T) * (sx * su)
    silu = lambda t: t / (1.0 + np.exp(-t))  # noqa: E731
    corners = np.stack([silu(gt + a * eg) * (ut + b * eu) for a in (-1, 1) for b in (-1, 1)]) / sh
    lo, hi = corners.min(axis=0), corners.max(axis=0)
    pad = 1e-5 * np.maximum(np.abs(lo), np.abs(hi)) + 1e-12
    _check_codes(hq, h / sh, lo - pad, hi + pad)
    del wg, wu
    wd = TABLE[codes[2].cpu().numpy().reshape(H, Fn)]
    want = (TABLE[hq] @ wd.T) * (sh * sd)
    got = y.cpu().numpy().reshape(M, H)[rows].astype(np.float64)
    assert np.all(np.abs(got - want) <= ATOL + RTOL * np.abs(want)), float(np.abs(got - want).max())
