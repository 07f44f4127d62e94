"""Pins `oracle.logfmt10_round_trip` (the LogFMT-10 codec of the reference's low-latency combine,
csrc/kernels/legacy/internode_ll.cu:556-712) by what the construction of the code grid fixes, none of it a
restatement of the oracle's formula:

  * a cast magnitude at or above the group's smallest grid point decodes to the NEAREST point (linear distance) of the
    grid {2^(log_amin + k * step), k = 0..510}: brute force over the grid, which catches a wrong rounding constant, an
    off-by-one in the codes or a swapped amax / amin;
  * the group's amax and (unclipped) amin come back unchanged: the two ends of the grid;
  * |decoded - x| <= (2^step - 1) / 2 * |x|, zeros stay zeros, signs survive, the map is monotone;
  * a chunk is left alone when any of its groups has amax >= 1 or a single magnitude (amin == amax), and the chunk is
    1024 channels for hidden % 1024 == 0, else 512.
"""
import numpy as np
import pytest
import torch

import routing_oracle as oracle


def _bf16(a):
    return torch.as_tensor(a, dtype=torch.float32).to(torch.bfloat16)


def _random_rows(seed, rows, hidden, scale):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn((rows, hidden), generator=g) * scale).to(torch.bfloat16)


def _grid(group):
    mag = group.double().abs().numpy()
    log_amax = np.log2(mag.max())
    log_amin = log_amax - 32 if mag.min() == 0 else max(np.log2(mag.min()), log_amax - 32)
    step = (log_amax - log_amin) / 510
    return np.exp2(log_amin + step * np.arange(511)), step


@pytest.mark.parametrize("seed,scale", [(0, 0.1), (1, 0.02), (2, 0.3), (3, 1e-3)])
def test_cast_values_decode_to_the_nearest_grid_point(seed, scale):
    x = _random_rows(seed, 4, 1024, scale).clamp(-0.99, 0.99)          # every group castable
    out = oracle.logfmt10_round_trip(x).double().numpy()
    xs = x.double().numpy()
    checked = 0
    for r in range(x.shape[0]):
        for g0 in range(0, 1024, 128):
            grid, step = _grid(x[r, g0:g0 + 128])
            for c in range(g0, g0 + 128):
                m = abs(xs[r, c])
                if m < grid[0]:
                    continue
                nearest = grid[np.argmin(np.abs(grid - m))]
                assert abs(abs(out[r, c]) - nearest) <= 1e-6 * nearest, (r, c, m, out[r, c], nearest)
                assert abs(abs(out[r, c]) - m) <= (2 ** step - 1) / 2 * m * (1 + 1e-6)
                assert np.sign(out[r, c]) == np.sign(xs[r, c])
                checked += 1
    assert checked > 3500


def test_ends_of_the_grid_survive():
    x = _random_rows(5, 2, 512, 0.2).clamp(-0.9, 0.9)
    out = oracle.logfmt10_round_trip(x)
    for r in range(2):
        for g0 in range(0, 512, 128):
            grp, dec = x[r, g0:g0 + 128].float(), out[r, g0:g0 + 128]
            hi, lo = grp.abs().argmax(), grp.abs().argmin()
            assert torch.isclose(dec[hi], grp[hi], rtol=1e-6, atol=0)
            if grp.abs()[lo] > grp.abs()[hi] * 2.0 ** -32:
                assert torch.isclose(dec[lo], grp[lo], rtol=1e-6, atol=0)


def test_zeros_signs_and_monotonicity():
    mags = torch.linspace(0.001, 0.9, 128)
    row = torch.cat([mags, -mags, mags * 0.5, mags.flip(0)])[None, :]
    row[0, 300] = 0.0
    x = _bf16(row)
    out = oracle.logfmt10_round_trip(x)[0]
    assert not torch.equal(out, x[0].float())                        # the chunk was cast
    assert float(out[300]) == 0.0
    assert bool((out[128:256] <= 0).all()) and bool((out[:128] >= 0).all())
    assert bool((out[:128][1:] >= out[:128][:-1]).all())             # monotone on an increasing ramp
    # literal: a group {0.5, 0.25, 0.25, ...} has a two-point grid 0.25 .. 0.5, both ends exact
    lit = torch.full((1, 512), 0.25)
    lit[0, ::2] = 0.5
    assert torch.equal(oracle.logfmt10_round_trip(_bf16(lit)), lit)


def test_chunks_that_are_left_alone():
    x = _random_rows(7, 3, 2048, 0.1).clamp(-0.9, 0.9)
    x[0, 1500] = 1.0                      # amax == 1 is not < 1: log_amax < 0 fails, the whole second chunk stays BF16
    x[1, 0:128] = 0.125                   # one magnitude only: log_amin == log_amax
    x[2, 1024:1152] = 0.0                 # an all-zero group: amax == 0, log_amin == log_amax == -inf
    out = oracle.logfmt10_round_trip(x)
    assert torch.equal(out[0, 1024:], x[0, 1024:].float()) and not torch.equal(out[0, :1024], x[0, :1024].float())
    assert torch.equal(out[1, :1024], x[1, :1024].float()) and not torch.equal(out[1, 1024:], x[1, 1024:].float())
    assert torch.equal(out[2, 1024:], x[2, 1024:].float())
    # 1536 channels are not a multiple of 1024: chunks of 512
    y = _random_rows(8, 1, 1536, 0.1).clamp(-0.9, 0.9)
    y[0, 600] = 2.0
    out = oracle.logfmt10_round_trip(y)
    assert torch.equal(out[0, 512:1024], y[0, 512:1024].float())
    assert not torch.equal(out[0, :512], y[0, :512].float()) and not torch.equal(out[0, 1024:], y[0, 1024:].float())


def test_clipped_range_and_calc_diff_bound():
    # a group spanning more than 2^32: values below amax * 2^-32 collapse to zero or the lowest grid point
    row = torch.full((1, 512), 0.5)
    row[0, 1::2] = 0.25                # every group holds two magnitudes, so the whole chunk is cast
    row[0, 5] = 2.0 ** -60
    row[0, 6] = 2.0 ** -33.4          # just under the clip point 2^-33: within half a step of the lowest grid point
    out = oracle.logfmt10_round_trip(_bf16(row))[0]
    assert float(out[5]) == 0.0 and float(out[0]) == 0.5
    assert float(out[6]) in (0.0, pytest.approx(2.0 ** -33, rel=1e-6))
    # the reference's acceptance bar for the combine that uses the codec (tests/legacy/test_low_latency.py:178-181)
    x = _random_rows(9, 64, 7168, 0.1)
    q = oracle.logfmt10_round_trip(x).double()
    ref = x.double()
    diff = 1 - 2 * (ref * q).sum() / ((ref * ref).sum() + (q * q).sum())
    assert 0 < float(diff) < 1e-5
