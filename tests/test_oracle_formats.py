"""Pins the oracle's byte and integer work: half / bfloat16 conversions against numpy over every bit pattern, the q8_0 /
q4_0 / GLM q8 quantizers against hand-derived known answers and an independent numpy statement of ggml's
quantize_row_q8_0_ref / quantize_row_q4_0_ref rules, the seeded generator against its definition, the split rules
against the reference's own figures."""
import numpy as np
import pytest

from oracle import orc


# ---- conversions -----------------------------------------------------------------------------------------------------
def test_h2f_every_bit_pattern():
    h = np.arange(65536, dtype=np.uint16)
    got, want = orc.h2f(h), h.view(np.float16).astype(np.float32)
    assert ((got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))).all()


def test_f2h_round_to_nearest_even():
    # every half, the float just below and above it, and the midpoints between neighbours (ties go to the even one)
    h = np.arange(0x7c00, dtype=np.uint16)
    f = h.view(np.float16).astype(np.float32)
    mid = ((f[:-1].astype(np.float64) + f[1:].astype(np.float64)) / 2).astype(np.float32)   # exact in float32
    xs = np.concatenate([f, -f, np.nextafter(f, np.float32(np.inf)), np.nextafter(f, np.float32(-np.inf)), mid, -mid,
                         np.array([65504, 65519.996, 65520, 1e9, np.inf, -np.inf, 2.0 ** -25, 2.0 ** -25 * 1.0000001, 2.0 ** -24 * 1.5, 0.0, -0.0], np.float32)])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    assert np.array_equal(orc.f2h(xs), want)
    rng = np.random.default_rng(1)
    r = (rng.standard_normal(2_000_000) * rng.choice([1e-7, 1e-5, 1e-3, 1.0, 300.0, 6e4], 2_000_000)).astype(np.float32)
    with np.errstate(over="ignore"):
        assert np.array_equal(orc.f2h(r), r.astype(np.float16).view(np.uint16))
    assert (orc.f2h(np.array([np.nan], np.float32)) & 0x7c00) == 0x7c00 and (orc.f2h(np.array([np.nan], np.float32)) & 0x3ff) != 0


def test_bf16_round_to_nearest_even():
    b = np.arange(65536, dtype=np.uint16)
    f = orc.bf2f(b)
    assert np.array_equal(f.view(np.uint32), b.astype(np.uint32) << 16)
    ok = ~np.isnan(f)
    assert np.array_equal(orc.f2bf(f[ok]), b[ok])                       # every bfloat16 maps to itself
    x = np.array([1.0, 1.0 + 2.0 ** -8, 1.0 + 2.0 ** -8 + 2.0 ** -20, 1.0 + 3 * 2.0 ** -8, 3.4e38, -2.5], np.float32)
    #             exact  tie -> even (1.0)  just above the tie -> up      tie -> even (up)   rounds to inf
    assert list(orc.f2bf(x)) == [0x3F80, 0x3F80, 0x3F81, 0x3F82, 0x7F80, 0xC020]
    rng = np.random.default_rng(2)
    r = rng.standard_normal(1_000_000).astype(np.float32)
    u = r.view(np.uint32)
    want = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    assert np.array_equal(orc.f2bf(r), want)


# ---- the generator -----------------------------------------------------------------------------------------------------
def _xorshift(seed, n):
    out, s, M = [], seed, (1 << 64) - 1
    for _ in range(n):
        s ^= s >> 12
        s ^= (s << 25) & M
        s ^= s >> 27
        out.append(((s * 0x2545F4914F6CDD1D) & M) >> 40)
    return np.array(out, np.uint64)


def test_generator_is_xorshift64star_box_muller():
    k = _xorshift(0xA11CE, 2000)
    assert np.array_equal(orc.uniform(0xA11CE, 2000), (k.astype(np.float64) / 2 ** 24).astype(np.float32))
    u1 = (k[0::2].astype(np.float64) + 1.0) / 2 ** 24
    u2 = k[1::2].astype(np.float64) / 2 ** 24
    r = np.sqrt(-2.0 * np.log(u1))
    z = np.empty(2000)
    z[0::2], z[1::2] = r * np.cos(2 * np.pi * u2), r * np.sin(2 * np.pi * u2)
    got = orc.randn(0xA11CE, (2000,), 0.5)
    assert np.abs(got - (0.5 * z).astype(np.float32)).max() <= 1e-6      # libm against numpy: last-bit differences only
    big = orc.randn(7, (1 << 20,))
    assert abs(big.mean()) < 5e-3 and abs(big.std() - 1.0) < 5e-3
    assert np.array_equal(orc.randn(7, (999,)), big[:999])               # an odd count is a prefix


# ---- q8_0 --------------------------------------------------------------------------------------------------------------
def _q8_0_numpy(x):
    """ggml quantize_row_q8_0_ref on blocks of 32: d = amax / 127, id = 1 / d, q = round-half-away(x * id)."""
    x = x.reshape(-1, 32).astype(np.float32)
    amax = np.abs(x).max(axis=1)
    d = (amax / np.float32(127.0)).astype(np.float32)
    idv = np.where(d != 0, np.float32(1.0) / np.where(d != 0, d, 1), 0).astype(np.float32)
    p = (x * idv[:, None]).astype(np.float32)
    q = (np.sign(p) * np.floor(np.abs(p) + np.float32(0.5))).astype(np.int8)
    return q, d.astype(np.float16)


def test_q8_0_known_answers():
    D, Hkv = 128, 1
    x = np.zeros((1, D), np.float32)
    x[0, 32:64] = np.arange(32) - 16           # amax 16 -> d = 16/127
    x[0, 64] = 127.0                            # amax 127 -> d = 1 exactly
    x[0, 65:96] = np.array([0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 126.5, -126.5] + [3.49999, -3.49999] + [0] * 21, np.float32)
    x[0, 96:128] = 1e-3
    kc, _ = orc.kv_store(1, x, x, Hkv, D, 1, 0)
    row = kc[0, 0]
    q = row[:D].view(np.int8)
    sc = row[D:].view(np.float16)
    assert (q[:32] == 0).all() and sc[0] == 0                              # a zero block: d = 0, id = 0
    assert q[64] == 127 and sc[2] == 1.0
    assert list(q[65:75]) == [1, -1, 2, -2, 3, -3, 127, -127, 3, -3]       # ties away from zero; 126.5 -> 127
    assert (q[96:128] == 127).all() and sc[3] == np.float16(np.float32(1e-3) / np.float32(127))
    qq, dd = _q8_0_numpy(x[0])
    assert np.array_equal(q, qq.ravel()) and np.array_equal(sc.view(np.uint16), dd.view(np.uint16))


@pytest.mark.parametrize("D", [128, 256])
def test_q8_0_matches_ggml_rule_on_random_rows(D):
    T, Hkv = 64, 3
    k = orc.randn(5, (T, Hkv * D), 2.0)
    v = orc.randn(6, (T, Hkv * D), 0.01)
    kc, vc = orc.kv_store(1, k, v, Hkv, D, T, 0)
    for src, c in ((k, kc), (v, vc)):
        q, d = _q8_0_numpy(src.reshape(T, Hkv, D).transpose(1, 0, 2))
        assert np.array_equal(c[:, :, :D].view(np.int8).reshape(-1, 32), q)
        assert np.array_equal(c[:, :, D:].view(np.uint16).reshape(-1), d.view(np.uint16))
    assert kc.shape[2] == D + D // 16 == {128: 136, 256: 272}[D]        # llm/qwen35/src/engine.rs:54-60
    # the widening read: (float) q * (float) half scale, exactly
    deq = orc.kv_dequant(kc, 1, D)
    want = kc[:, :, :D].view(np.int8).astype(np.float32) * np.repeat(kc[:, :, D:].view(np.float16).astype(np.float32), 32, axis=2)
    assert np.array_equal(deq, want)


# ---- q4_0 --------------------------------------------------------------------------------------------------------------
def _q4_0_numpy(x):
    """ggml quantize_row_q4_0_ref: the value of the largest magnitude (first of a tie) / -8; q = min(15, trunc(x id + 8.5));
    byte j = value j | value j + 16 << 4."""
    x = x.reshape(-1, 32).astype(np.float32)
    at = np.abs(x).argmax(axis=1)                 # numpy's argmax keeps the first maximum
    m = x[np.arange(len(x)), at]
    d = (m / np.float32(-8.0)).astype(np.float32)
    idv = np.where(d != 0, np.float32(1.0) / np.where(d != 0, d, 1), 0).astype(np.float32)
    qv = np.minimum(15, ((x * idv[:, None]).astype(np.float32) + np.float32(8.5)).astype(np.float32).astype(np.int32))
    by = (qv[:, :16] | (qv[:, 16:] << 4)).astype(np.uint8)
    return by, d.astype(np.float16)


def test_q4_0_known_answers_and_rule():
    D, Hkv = 128, 1
    x = np.zeros((1, D), np.float32)
    x[0, 32:64] = np.where(np.arange(32) % 2 == 0, 2.0, -2.0)      # tie of magnitudes: the first (+2) -> d = -0.25
    x[0, 64:96] = np.where(np.arange(32) % 2 == 0, -2.0, 2.0)      # the first is -2 -> d = +0.25
    x[0, 96:128] = np.linspace(-1, 1, 32)
    kc, _ = orc.kv_store(2, x, x, Hkv, D, 1, 0)
    row = kc[0, 0]
    assert row.size == D // 2 + D // 16 == 72
    sc = row[D // 2:].view(np.float16)
    assert sc[0] == 0 and (row[:16] == 0x88).all()                  # zero block: id = 0 -> q = trunc(8.5) = 8 everywhere
    assert sc[1] == np.float16(-0.25) and sc[2] == np.float16(0.25)
    # +2 with d = -0.25: x id = -8 -> q 0; -2 -> +8 -> 16.5 -> clipped to 15. value j low nibble, j + 16 high nibble
    assert (row[16:32] == np.where(np.arange(16) % 2 == 0, 0x00, 0xFF)).all()
    assert (row[32:48] == np.where(np.arange(16) % 2 == 0, 0x00, 0xFF)).all()
    by, d = _q4_0_numpy(x[0])
    assert np.array_equal(row[:D // 2], by.ravel()) and np.array_equal(sc.view(np.uint16), d.view(np.uint16))
    k = orc.randn(9, (40, 256), 1.5)
    kc, _ = orc.kv_store(2, k, k, 1, 256, 40, 0)
    by, d = _q4_0_numpy(k)
    assert np.array_equal(kc[0, :, :128].reshape(-1, 16), by) and np.array_equal(kc[0, :, 128:].view(np.uint16).ravel(), d.view(np.uint16))
    # the widening read: nibble - 8 times the half scale; value j < 16 in the low nibble of byte j
    deq = orc.kv_dequant(kc, 2, 256)[0]
    nib = np.concatenate([by & 15, by >> 4], axis=1).astype(np.float32) - 8
    assert np.array_equal(deq.reshape(-1, 32), nib * d.astype(np.float32)[:, None])


# ---- GLM q8 latent rows ---------------------------------------------------------------------------------------------------
def test_glm_q8row_scale_rounded_first_and_clamped():
    L = 64
    x = np.zeros((1, L), np.float32)
    x[0, :32] = np.linspace(-1, 1, 32) * 0.7
    x[0, 32:] = 1000.0 + np.arange(32)          # half(amax / 127) rounds DOWN here, so x / d can exceed 127: clamped
    y = orc.glm_to_q8row(x, L)
    sc = y[0, :4].view(np.float16)
    q = y[0, 4:].view(np.int8)
    assert y.shape[1] == L // 32 * 2 + L
    for b in range(2):
        xb = x[0, 32 * b:32 * b + 32]
        dh = np.float16(np.float32(np.abs(xb).max()) / np.float32(127))
        assert sc[b] == dh
        p = xb * (np.float32(1) / np.float32(dh))
        want = np.clip(np.sign(p) * np.floor(np.abs(p) + np.float32(0.5)), -127, 127)
        assert np.array_equal(q[32 * b:32 * b + 32], want.astype(np.int8))
    assert q.max() == 127 and (np.abs(x[0, 32:] / np.float32(sc[1])) > 127).any()


# ---- Walsh-Hadamard ---------------------------------------------------------------------------------------------------------
def test_fwht32_is_the_normalized_hadamard_matrix():
    H = np.array([[1.0]])
    for _ in range(5):
        H = np.block([[H, H], [H, -H]])
    x = orc.randn(4, (3, 64))
    got = orc.fwht32(x)
    want = np.concatenate([x[:, :32].astype(np.float64) @ H, x[:, 32:].astype(np.float64) @ H], axis=1) / np.sqrt(32)
    assert np.abs(got - want).max() < 1e-5
    assert np.abs(orc.fwht32(got) - x).max() < 1e-5          # its own inverse


# ---- split rules ---------------------------------------------------------------------------------------------------------------
def test_reference_split_rules():
    L = orc.lib()
    # the XMX decode kernels' splits at the BASELINE shapes (kernels/llm/qwen35/silo/attn.cpp:321-331)
    assert (L.orc_dec_split(4096, 8), L.orc_dec_splits(4096, 8)) == (64, 64)
    assert (L.orc_dec_split(65537, 4), L.orc_dec_splits(65537, 4)) == (576, 114)
    assert (L.orc_dec_split(131072, 4), L.orc_dec_splits(131072, 4)) == (1024, 128)
    assert L.orc_dec_split(1, 8) == 64 and L.orc_dec_splits(64, 8) == 1 and L.orc_dec_splits(65, 8) == 2
    assert L.orc_q35_attn_decode_scratch(1, 32, 8, 128, 4095) == 32 * 64 * 130
    assert L.orc_q35_attn_decode_scratch(1, 32, 8, 128, 10) == 0
    # the exact kernels': multiples of 32, only decode rows split (q35: one row; mg: up to 16)
    assert L.orc_q35_split_keys(1, 4096, 8) == 64 and L.orc_q35_split_keys(2, 4096, 8) == 4096
    assert L.orc_mg_split_keys(16, 4096, 8) == 64 and L.orc_mg_split_keys(17, 4096, 8) == 4096
    assert L.orc_mg_splits(1, 100, 1) == 4 and L.orc_mg_splits(1, 32, 1) == 1
    assert L.orc_mg_seen(4, 100, 0, 1) == 104 and L.orc_mg_seen(4, 100, 50, 1) == 50 and L.orc_mg_seen(4, 100, 50, 0) == 104 - 51
