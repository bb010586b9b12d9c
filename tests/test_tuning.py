"""The numbers that choose between kernels are one dataclass; a kernel table takes a changed set."""
from dataclasses import fields

import pytest

from servelab_amd.kernels.tuning import Tuning


def test_every_choice_lands_on_the_table_under_its_upper_case_name():
    class Table:
        pass
    t = Table()
    Tuning(few_wave_us=2.5, wide_min_m=33).apply(t)
    assert t.FEW_WAVE_US == 2.5 and t.WIDE_MIN_M == 33
    assert t.NARROW_ATTENTION_WORKGROUPS == Tuning().narrow_attention_workgroups
    assert {n for n in vars(t)} == {f.name.upper() for f in fields(Tuning)}


@pytest.mark.gpu
def test_a_kernel_table_with_other_choices_gives_the_same_numbers():
    """Choices move work between kernels, never the result beyond rounding: a decode attention
    split into few wavefronts or many, a product on the one-tile or the LDS-staged kernel."""
    import torch
    from servelab_amd.kernels import HipOps
    a = HipOps(torch.bfloat16, "cuda:0")
    b = HipOps(torch.bfloat16, "cuda:0", tuning=Tuning(few_wave_us=20.0, mid_min_elements=1 << 40,
                                                       mid_min_elements_many=1 << 40, resident_min_rounds=1 << 20))
    assert b.FEW_WAVE_US == 20.0 and a.FEW_WAVE_US == Tuning().few_wave_us
    assert b._decode_shares(32, 64, 128, 128) < a._decode_shares(32, 64, 128, 128)
    g = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn(40, 1024, device="cuda", generator=g).bfloat16()
    w = (torch.randn(12288, 1024, device="cuda", generator=g) * 0.03).bfloat16()
    wa, wb = a.prepare_weight(w), b.prepare_weight(w)
    assert a._takes_mid(40, 12288, 1024) and not b._takes_mid(40, 12288, 1024)
    ya, yb = a.linear(x, wa, None).float(), b.linear(x, wb, None).float()
    ref = x.float() @ w.float().T
    assert (ya - ref).abs().max() < 2 ** -6 * ref.abs().max()
    assert (yb - ref).abs().max() < 2 ** -6 * ref.abs().max()
