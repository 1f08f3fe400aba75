"""CPU checks of the add_to_fp8 oracle: a case worked by hand and the structure of the identity."""

import torch

from oracle import arithmetic as oarith, cast as ocast, fp8


def test_hand_worked_case():
    # E4M3 codes for 1.0, -2.0, 0.5, 0 with scale 4 (stored value = real * 4): real = [0.25, -0.5, 0.125, 0]
    q = fp8.encode(torch.tensor([1.0, -2.0, 0.5, 0.0]), fp8.E4M3)
    meta = ocast.new_meta()
    meta['scale'], meta['scale_inv'] = torch.tensor(4.0), torch.tensor(0.25)
    other = torch.tensor([0.75, 0.5, 1.875, -3.0])
    out = oarith.add_to_fp8(q, meta, fp8.E4M3, other)
    # sum = [1, 0, 2, -3]; amax 3 -> scale 2**floor(log2(448/3)) = 128; payload = sum * 128
    assert meta['amax'][0].item() == 3.0 and meta['scale'].item() == 128.0 and meta['scale_inv'].item() == 1 / 128
    assert torch.equal(fp8.decode(out, fp8.E4M3), torch.tensor([128.0, 0.0, 256.0, -384.0]))


def test_sum_is_rounded_to_the_dtype_of_other():
    # 1 + 2**-9 is not a bf16 (8 significand bits): the sum must round to 1 before the amax is taken
    q = fp8.encode(torch.tensor([1.0]), fp8.E5M2)
    meta = ocast.new_meta()
    out = oarith.add_to_fp8(q, meta, fp8.E5M2, torch.tensor([2.0**-9], dtype=torch.bfloat16))
    assert meta['amax'][0].item() == 1.0 and meta['scale'].item() == 32768.0
    assert fp8.decode(out, fp8.E5M2).item() == 32768.0
