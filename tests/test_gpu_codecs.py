"""Device element codecs against the CPU oracle, bit for bit, on inputs chosen to hit every
rounding decision (all codes, every tie, saturation edges, denormals) plus random bits."""
import numpy as np
import pytest

from rivoli_amd import hip
from tests.gpu_util import back, dev, dzeros, torch_cuda
from tests.test_oracle_codecs import all_e4m3_values

pytestmark = pytest.mark.gpu


def encode_probe_set():
    vals = all_e4m3_values()[:0x7F].astype(np.float32)
    mids = ((all_e4m3_values()[:0x7E] + all_e4m3_values()[1:0x7F]) / 2).astype(np.float32)
    near = np.concatenate([np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e9))])
    rng = np.random.default_rng(0xE4)
    rand_bits = rng.integers(0, 2 ** 32, 1 << 22, dtype=np.uint64).astype(np.uint32).view(np.float32)
    band = np.exp(rng.uniform(np.log(2.0 ** -13), np.log(1000.0), 1 << 22)).astype(np.float32)
    edge = np.array([0.0, 447.99, 448.0, 464.0, 480.0, 1e30, np.inf, 2.0 ** -10, 2.0 ** -6,
                     np.nextafter(np.float32(2.0 ** -10), np.float32(0)),
                     np.nextafter(np.float32(2.0 ** -6), np.float32(0)),
                     np.nextafter(np.float32(448.0), np.float32(0)), 1e-45, 1e-39, np.nan],
                    np.float32)
    x = np.concatenate([vals, mids, near, band, edge])
    return np.concatenate([x, -x, rand_bits])


def test_e4m3_encode_matches_oracle(oracle):
    x = encode_probe_set()
    out = dzeros(x.size)
    hip.launch_codec_e4m3_encode(dev(x), out, x.size)
    got, want = back(out), oracle.f32_to_e4m3(x)
    bad = np.flatnonzero(got != want)
    assert bad.size == 0, [(x[i], hex(got[i]), hex(want[i])) for i in bad[:8]]
    # the probe really contains the subnormal ties that separate half-away from nearest-even
    q = np.float32(2.0 ** -10)
    assert np.isin(np.array([1, 5, 9, 13], np.float32) * q, x).all()


@pytest.mark.parametrize("quarter", range(4))
def test_e4m3_encode_every_f32_bit_pattern(oracle, quarter):
    """All 2^32 inputs, a quarter per case, in pieces of 2^26 generated on the device."""
    torch = torch_cuda()
    piece = 1 << 26
    out = dzeros(piece)
    for k in range(quarter * 16, quarter * 16 + 16):
        base = k * piece
        wide = torch.arange(base, base + piece, dtype=torch.int64, device="cuda")
        bits = torch.where(wide >= 1 << 31, wide - (1 << 32), wide).to(torch.int32)
        hip.launch_codec_e4m3_encode(bits.view(torch.uint8), out, piece)
        host = (np.arange(piece, dtype=np.uint32) + np.uint32(base)).view(np.float32)
        got, want = back(out), oracle.f32_to_e4m3(host)
        bad = np.flatnonzero(got != want)
        assert bad.size == 0, [(hex(base + int(i)), hex(got[i]), hex(want[i])) for i in bad[:8]]


def test_e4m3_dequant_matches_oracle_for_every_code(oracle):
    codes = np.arange(256, dtype=np.uint8)
    finite = (codes & 0x7F) != 0x7F
    scales = [1.0, 0.0022321429, 3.5e-3, 1e-30, 7e-42, 2.5e35, 448.0, 2.0 ** -140, -1.5]
    for scale in scales:
        scale = np.float32(scale)
        out = dzeros(512)
        hip.launch_codec_e4m3_dequant_bf16(dev(codes), float(scale), out, 256)
        got = back(out, np.uint16)
        want = oracle.f32_to_bf16(oracle.e4m3_to_f32(codes) * scale)
        assert np.array_equal(got[finite], want[finite]), float(scale)
        # the two NaN codes stay NaN
        assert all((int(g) & 0x7F80) == 0x7F80 and (int(g) & 0x7F) for g in got[~finite])


def test_bf16_encode_matches_oracle(oracle):
    rng = np.random.default_rng(0xBF16)
    bits = rng.integers(0, 2 ** 32, 1 << 23, dtype=np.uint64).astype(np.uint32)
    # every exact tie and its neighbours for a spread of exponents, both parities
    hi = rng.integers(0, 2 ** 16, 1 << 16, dtype=np.uint64).astype(np.uint32) << 16
    ties = np.concatenate([hi | 0x8000, hi | 0x7FFF, hi | 0x8001])
    x = np.concatenate([bits, ties]).view(np.float32)
    x = x[~np.isnan(x)]
    out = dzeros(x.size * 2)
    hip.launch_codec_bf16_encode(dev(x), out, x.size)
    assert np.array_equal(back(out, np.uint16), oracle.f32_to_bf16(x))
    nan_out = dzeros(2)
    hip.launch_codec_bf16_encode(dev(np.array([np.nan], np.float32)), nan_out, 1)
    g = int(back(nan_out, np.uint16)[0])
    assert (g & 0x7F80) == 0x7F80 and (g & 0x7F)


def test_codec_launcher_guards():
    buf = dzeros(16)
    for fn, args in ((hip.launch_codec_e4m3_encode, (buf, buf, 0)),
                     (hip.launch_codec_e4m3_encode, (None, buf, 4)),
                     (hip.launch_codec_bf16_encode, (buf, None, 4)),
                     (hip.launch_codec_e4m3_dequant_bf16, (buf, 1.0, buf, -1))):
        with pytest.raises(hip.LaunchError) as e:
            fn(*args)
        assert e.value.code == 1001
