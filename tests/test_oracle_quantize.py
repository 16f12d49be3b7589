"""Pins of the quantize / dequantize oracle (CPU only).

Each test checks the oracle against something it did not come from: torch's own
float8_e4m3fn and bf16 casts (exhaustively), closed forms, the reference's
known answers (tests/golden), or an invariant of the scheme.  The C port and
the eager restatement are also held to each other bit for bit.
"""

import math

import pytest
import torch

from oracle import cport, eager

BLOCK = 4


def all_bf16() -> torch.Tensor:
    """Every bf16 bit pattern as a bf16 tensor (65 536 values)."""
    return torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)


def bits32(t: torch.Tensor) -> torch.Tensor:
    return t.contiguous().view(torch.int32)


def test_e4m3_conversion_matches_torch_for_every_bf16_value_and_scale():
    """The C E4M3FN rounding (written from the format definition) equals
    torch's cast on all bf16 inputs times a spread of scales, including values
    that land on subnormals, ties and the non-saturating overflow."""
    values = all_bf16().float()
    for scale in (1.0, 0.5, 3.0, 448.0, 2.0**-9, 1.7e-3, 13.25):
        scaled = values * scale
        want = scaled.to(torch.float8_e4m3fn).view(torch.uint8)
        got = torch.tensor([cport.f32_to_e4m3fn(v) for v in scaled.tolist()], dtype=torch.uint8)
        nan = scaled.isnan()
        assert torch.equal(got[~nan], want[~nan]), f"scale {scale}"
        assert ((got[nan] & 0x7F) == 0x7F).all()


def test_e4m3_decode_matches_torch_for_every_byte():
    table = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(torch.float8_e4m3fn).float()
    for byte in range(256):
        got = cport.e4m3fn_to_f32(byte)
        want = table[byte].item()
        assert (math.isnan(got) and math.isnan(want)) or got == want, byte


def test_bf16_rounding_matches_torch():
    gen = torch.Generator().manual_seed(5)
    x = torch.randn(20000, generator=gen) * torch.logspace(-30, 30, 20000)
    want = x.bfloat16().view(torch.int16).to(torch.int32) & 0xFFFF
    got = torch.tensor([cport.lib().fso_scalar_f32_to_bf16(v) for v in x.tolist()], dtype=torch.int32)
    assert torch.equal(got, want)


def test_constant_tile_closed_form():
    """A tile of constant c: amax = |c|, every byte is +-448 (0x7E / 0xFE) and
    the stored scale is fp32(1 / fp32(448 / |c|))."""
    for c in (0.02, -3.0, 1.0, 7.25e-5, 448.0, 1e30):
        w = torch.full((8, 8), c).bfloat16()
        q, s = cport.quantize_blockwise(w, BLOCK)
        assert (q == (0x7E if c > 0 else 0xFE)).all()
        amax = abs(w[0, 0].item())
        scale32 = torch.tensor(448.0 / amax, dtype=torch.float64).to(torch.float32)
        want = (torch.tensor(1.0, dtype=torch.float32) / scale32).expand(2, 2)
        assert torch.equal(bits32(s), bits32(want))


def test_stored_scale_is_reciprocal_of_rounded_scale_not_amax_over_448():
    """amax/448 differs from 1/fp32(448/amax) in the last bit for many amax;
    the oracle must follow the latter."""
    amaxes = all_bf16()[0x2C00:0x7F80:37].float()  # above the 1e-12 floor, below inf
    differing = 0
    for amax in amaxes.tolist():
        w = torch.zeros(4, 4)
        w[1, 2] = amax
        _, s = cport.quantize_blockwise(w.bfloat16(), BLOCK)
        scale32 = (torch.tensor(448.0, dtype=torch.float64) / amax).to(torch.float32)
        want = torch.tensor(1.0, dtype=torch.float32) / scale32
        assert s.view(torch.int32).item() == want.view(torch.int32).item()
        naive = torch.tensor(amax / 448.0, dtype=torch.float64).to(torch.float32)
        differing += int(naive.view(torch.int32).item() != want.view(torch.int32).item())
    assert differing > len(amaxes) // 10  # the distinction is real, not vacuous


def test_zero_tile_eps_constants(golden):
    g = golden["quant_eps_constants"]
    q, s = cport.quantize_blockwise(torch.zeros(4, 4).bfloat16(), BLOCK)
    assert (q == 0).all()
    assert s.view(torch.int32).item() == int(g["zero_tile_recip_bits_bf16_input"], 16)
    _, s32 = cport.quantize_blockwise(torch.zeros(4, 4), BLOCK)
    assert s32.view(torch.int32).item() == int(g["zero_tile_recip_bits_fp32_input"], 16)
    _, s_forced = cport.quantize_blockwise(torch.zeros(4, 4).bfloat16(), BLOCK, eps_mode=cport.EPS_FP32)
    assert s_forced.view(torch.int32).item() == int(g["zero_tile_recip_bits_fp32_input"], 16)
    # The eager restatement lands on the same two constants.
    _, e = eager.quantize_blockwise(torch.zeros(4, 4).bfloat16(), BLOCK)
    assert e.view(torch.int32).item() == int(g["zero_tile_recip_bits_bf16_input"], 16)
    _, e32 = eager.quantize_blockwise(torch.zeros(4, 4), BLOCK)
    assert e32.view(torch.int32).item() == int(g["zero_tile_recip_bits_fp32_input"], 16)


def test_known_answer_param_dtype_cast(golden):
    """fp32 master 0.25 with one 1.001 quantized as bf16: amax rounds to 1.0,
    scale 448, bytes e4m3(112) except the outlier 0x7E; quantizing the fp32
    values directly gives a different scale."""
    g = golden["fp8_quantizes_param_dtype"]
    w = torch.full((4, 4), g["fill"], dtype=torch.float32)
    w[tuple(g["outlier_index"])] = g["outlier"]
    q, s = cport.quantize_blockwise(w, g["block"], cast_to_bf16=True)
    fill_byte = torch.tensor(g["fill_byte_is_e4m3_of"]).to(torch.float8_e4m3fn).view(torch.uint8).item()
    want = torch.full((4, 4), fill_byte, dtype=torch.uint8)
    want[0, 0] = g["outlier_byte"]
    assert torch.equal(q, want)
    assert s.item() == torch.tensor(1.0 / 448.0, dtype=torch.float32).item()
    q2, s2 = cport.quantize_blockwise(w.bfloat16(), g["block"])
    assert torch.equal(q, q2) and torch.equal(bits32(s), bits32(s2))
    _, s_fp32 = cport.quantize_blockwise(w, g["block"])
    assert not torch.equal(bits32(s), bits32(s_fp32))


def test_power_of_two_amax_reduces_to_plain_cast():
    """With amax = 2^k the scale 448 * 2^-k is exact, so q must equal torch's
    cast of x * scale for every bf16 x with |x| <= amax (brute force)."""
    for k in (0, -6, 5):
        amax = 2.0**k
        values = all_bf16().float()
        values = values[values.abs() <= amax]
        values = values[: (values.numel() // 4) * 4]
        w = values.view(-1, 4).clone()
        w[0::4, 0] = amax  # every 4-row tile carries the amax
        q, s = cport.quantize_blockwise(w.bfloat16(), BLOCK)
        want = (w.bfloat16().float() * (448.0 / amax)).to(torch.float8_e4m3fn).view(torch.uint8)
        usable = (w.shape[0] // 4) * 4
        assert torch.equal(q[:usable], want[:usable])
        assert (s[: usable // 4] == amax / 448.0).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_c_port_equals_eager_on_random_data_with_outliers(dtype):
    gen = torch.Generator().manual_seed(11)
    for shape, block, std in (((64, 48), 4, 0.02), ((130, 136), 128, 0.006), ((9, 32), 2, 1.0), ((257, 129), 128, 0.02)):
        w = torch.randn(shape, generator=gen) * std
        mask = torch.rand(shape, generator=gen) < 0.01
        w[mask] *= 50
        w[: min(block, shape[0]), : min(block, shape[1])] = 0
        w = w.to(dtype)
        cq, cs = cport.quantize_blockwise(w, block)
        eq, es = eager.quantize_blockwise(w, block)
        assert torch.equal(cq, eq.view(torch.uint8))
        assert torch.equal(bits32(cs), bits32(es))


def test_partial_block_shapes_of_the_reference_test(golden):
    g = golden["partial_block_shapes"]
    for shape in g["shapes"]:
        torch.manual_seed(g["seed"])
        w = torch.randn(shape, dtype=torch.bfloat16)
        cq, cs = cport.quantize_blockwise(w, g["block"])
        eq, es = eager.quantize_blockwise(w, g["block"])
        assert cq.shape == tuple(shape) and cs.shape == (-(-shape[0] // 4), -(-shape[1] // 4))
        assert torch.equal(cq, eq.view(torch.uint8)) and torch.equal(bits32(cs), bits32(es))


def test_quantize_then_gather_equals_gather_then_quantize():
    """Cutting a matrix on tile-row boundaries and quantizing the pieces gives
    the same bytes and scales as quantizing the whole matrix, for any number
    of pieces (the property behind the FP8 all-gather)."""
    gen = torch.Generator().manual_seed(2)
    w = (torch.randn(40, 24, generator=gen) * 0.02).bfloat16()
    whole_q, whole_s = cport.quantize_blockwise(w, BLOCK)
    for pieces in (1, 2, 3, 8):
        bounds = sorted({0, 40, *[4 * ((10 * i) // pieces) for i in range(1, pieces)]})
        qs, ss = [], []
        for lo, hi in zip(bounds, bounds[1:]):
            q, s = cport.quantize_blockwise(w[lo:hi], BLOCK)
            qs.append(q)
            ss.append(s)
        assert torch.equal(torch.cat(qs), whole_q)
        assert torch.equal(bits32(torch.cat(ss)), bits32(whole_s))


def test_nan_and_inf_tiles():
    w = torch.ones(8, 4).bfloat16()
    w[0, 0] = float("nan")
    w[5, 1] = float("inf")
    q, s = cport.quantize_blockwise(w, BLOCK)
    assert ((q[:4] & 0x7F) == 0x7F).all() and math.isnan(s[0, 0].item())  # NaN poisons its tile
    # amax = inf: scale 0, finite values become zero, inf * 0 is NaN, stored scale inf
    assert math.isinf(s[1, 0].item())
    assert (q[5, 1] & 0x7F) == 0x7F
    rest = q[4:].clone()
    rest[1, 1] = 0
    assert (rest == 0).all()
    eq, es = eager.quantize_blockwise(w, BLOCK)
    assert torch.equal(eq.view(torch.uint8)[4:], q[4:])


def test_strided_rows_are_supported():
    gen = torch.Generator().manual_seed(3)
    parent = (torch.randn(16, 20, generator=gen)).bfloat16()
    view = parent[:, 2:10]
    q, s = cport.quantize_blockwise(view, BLOCK)
    q2, s2 = cport.quantize_blockwise(view.contiguous(), BLOCK)
    assert torch.equal(q, q2) and torch.equal(bits32(s), bits32(s2))


# ------------------------------------------------------------------ dequant
def test_dequant_known_answer_flat(golden):
    g = golden["dequant_flat"]
    fp8 = torch.arange(128, dtype=torch.bfloat16).reshape(g["shape"]).to(torch.float8_e4m3fn)
    scale = torch.full(g["scale_shape"], g["scale"], dtype=torch.float32)
    want = fp8.float() * g["scale"]
    assert torch.equal(cport.dequant_blockwise(fp8.view(torch.uint8), scale, g["block"], torch.float32), want)
    assert torch.equal(eager.dequant_blockwise(fp8, scale, g["block"], torch.float32), want)
    assert torch.equal(cport.dequant_blockwise(fp8.view(torch.uint8), scale, g["block"]), want.bfloat16())


def test_dequant_known_answer_stacked(golden):
    g = golden["dequant_stacked"]
    fp8 = torch.arange(96, dtype=torch.bfloat16).reshape(g["shape"]).to(torch.float8_e4m3fn)
    scale = torch.tensor(g["scales"], dtype=torch.float32)
    per_elem = scale.repeat_interleave(g["block"], 0).repeat_interleave(g["block"], 1)
    want = fp8.float() * per_elem.view(g["shape"])
    flat = fp8.flatten(0, -2)
    got = cport.dequant_blockwise(flat.view(torch.uint8), scale, g["block"], torch.float32).view(g["shape"])
    assert torch.equal(got, want)
    assert torch.equal(eager.dequant_blockwise(flat, scale, g["block"], torch.float32).view(g["shape"]), want)


def test_dequant_every_byte_and_bf16_rounding():
    data = torch.arange(256, dtype=torch.int32).to(torch.uint8).repeat(2).view(16, 32)
    gen = torch.Generator().manual_seed(9)
    scale = torch.rand(4, 8, generator=gen) * 3e-3
    c = cport.dequant_blockwise(data, scale, 4)
    e = eager.dequant_blockwise(data.view(torch.float8_e4m3fn), scale, 4)
    finite = ~e.isnan()
    assert torch.equal(c.view(torch.int16)[finite], e.view(torch.int16)[finite])
    assert c.isnan().equal(e.isnan())


def test_quantize_dequantize_round_trip_error_bound():
    """|dequant(quant(x)) - x| <= amax * 2^-4 per tile (3 mantissa bits plus
    the subnormal floor), a property independent of any implementation."""
    gen = torch.Generator().manual_seed(4)
    w = (torch.randn(64, 64, generator=gen) * 0.02).bfloat16()
    q, s = cport.quantize_blockwise(w, 16)
    back = cport.dequant_blockwise(q, s, 16, torch.float32)
    tiles = w.float().view(4, 16, 4, 16).abs().amax(dim=(1, 3))
    bound = tiles.repeat_interleave(16, 0).repeat_interleave(16, 1) / 16
    assert ((back - w.float()).abs() <= bound).all()


@pytest.mark.parametrize("shape,block", [((12, 6), 4), ((130, 129), 128), ((64, 64), 16)])
def test_eager_restatement_on_fp16_input(shape, block):
    """What the reference's arithmetic gives on fp16: fp16 to fp32 is exact and
    no nonzero fp16 amax lies under the 1e-12 floor, so every tile with a
    nonzero amax equals the C quantization of the upcast values (pinned above);
    the floor itself rounds to 0 in fp16, so an all-zero tile gets scale inf,
    stored reciprocal 0 and NaN bytes (0 x inf)."""
    gen = torch.Generator().manual_seed(shape[0] + block)
    w = (torch.randn(shape, generator=gen) * 0.05).half()
    w[0, 0], w[-1, -1] = 6.1e-5, 65504.0
    q, s = eager.quantize_blockwise(w, block)
    cq, cs = cport.quantize_blockwise(w.float(), block)
    assert torch.equal(q.view(torch.uint8), cq) and torch.equal(s.view(torch.int32), cs.view(torch.int32))
    assert torch.tensor(1e-12).half().item() == 0.0
    w[:block, :block] = 0
    q, s = eager.quantize_blockwise(w, block)
    cq, cs = cport.quantize_blockwise(w.float(), block)
    tile = torch.zeros(shape, dtype=torch.bool)
    tile[:block, :block] = True
    assert s[0, 0].item() == 0.0 and ((q.view(torch.uint8)[tile] & 0x7F) == 0x7F).all()
    assert torch.equal(q.view(torch.uint8)[~tile], cq[~tile])
    assert torch.equal(s.view(torch.int32).view(-1)[1:], cs.view(torch.int32).view(-1)[1:])
    assert cs[0, 0].view(torch.int32).item() == 0x2720D7C5 and (cq[tile] == 0).all()  # the fp32 floor keeps the tile finite
