"""Pins for oracle.rope (restating inf_llm/attention/rope.py): closed form and invariants."""
import math

import torch

from oracle.rope import RopeOracle


def _complex_fp64(x, positions, base, scale=1.0):
    D = x.shape[-1]
    half = D // 2
    inv = torch.tensor([base ** (-2.0 * i / D) for i in range(half)], dtype=torch.float64)
    out = torch.empty_like(x, dtype=torch.float64)
    for r, p in enumerate(positions):
        for i in range(half):
            z = complex(float(x[..., r, i]), float(x[..., r, i + half])) * complex(
                math.cos(p * scale * inv[i]), math.sin(p * scale * inv[i]))
            out[..., r, i], out[..., r, i + half] = z.real, z.imag
    return out


def test_matches_fp64_complex_rotation():
    torch.manual_seed(0)
    rope = RopeOracle(16, base=10000)
    x = torch.randn(7, 16)
    pos = [0, 1, 2, 5, 17, 100, 333]
    got = rope.rotate(x, pos)
    want = _complex_fp64(x, pos, 10000)
    assert torch.allclose(got.double(), want, atol=2e-5)


def test_distance_scale_multiplies_position():
    torch.manual_seed(1)
    x = torch.randn(4, 8)
    a = RopeOracle(8, base=500, distance_scale=0.5).rotate(x, [0, 2, 4, 6])
    b = RopeOracle(8, base=500).rotate(x, [0, 1, 2, 3])
    assert torch.allclose(a, b, atol=1e-6)


def test_position_zero_is_identity_and_norm_is_kept():
    torch.manual_seed(2)
    rope = RopeOracle(32, base=1e6)
    x = torch.randn(2, 3, 9, 32)
    assert torch.equal(rope.rotate(x, [0] * 9), x)
    y = rope.rotate(x, list(range(40, 49)))
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), atol=1e-5)


def test_inner_product_depends_on_relative_position_only():
    torch.manual_seed(3)
    rope = RopeOracle(32, base=1e4)
    q, k = torch.randn(1, 32), torch.randn(1, 32)
    ref = (rope.rotate(q, [9]) * rope.rotate(k, [4])).sum()
    for shift in (1, 13, 200):
        got = (rope.rotate(q, [9 + shift]) * rope.rotate(k, [4 + shift])).sum()
        assert abs(float(got - ref)) < 2e-4
    # sign convention: swapping which side is ahead changes the value
    other = (rope.rotate(q, [4]) * rope.rotate(k, [9])).sum()
    assert abs(float(other - ref)) > 1e-3


def test_window_and_one_angle_positions():
    torch.manual_seed(4)
    rope = RopeOracle(16, base=1e4)
    q, k = torch.randn(1, 2, 3, 16), torch.randn(1, 1, 10, 16)
    qr, kr = rope.window(q, k)
    assert torch.equal(qr, rope.rotate(q, [7, 8, 9]))
    assert torch.equal(kr, rope.rotate(k, list(range(10))))
    # one_angle(x, n) puts every row at position n-1
    oa = rope.one_angle(q, 8)
    assert torch.equal(oa, rope.rotate(q, [7, 7, 7]))
    assert torch.equal(oa[..., 0, :], qr[..., 0, :])


def test_low_precision_input_is_rotated_in_fp32_and_cast_back():
    torch.manual_seed(5)
    rope = RopeOracle(16, base=1e4)
    x = torch.randn(5, 16).bfloat16()
    y = rope.rotate(x, [3] * 5)
    assert y.dtype == torch.bfloat16
    assert torch.equal(y, rope.rotate(x.float(), [3] * 5).bfloat16())
