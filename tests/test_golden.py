"""The committed known-answer vectors (tests/golden/*.json, written by
tests/golden/make_fixtures.py from the index-arithmetic replay of the reference
kernels) against the oracle on the CPU and against the HIP kernels on the GPU."""
import json
import os

import pytest
import torch

from oracle import eager

HERE = os.path.dirname(os.path.abspath(__file__))


def _load(name):
    with open(os.path.join(HERE, "golden", name)) as f:
        return json.load(f)


PACK = _load("pack_kat.json")
MATH = _load("math_kat.json")


def test_reference_test_constants():
    ref = PACK["reference_test"]
    assert ref["seq_lens"] == [24, 127, 31, 65, 24, 127, 31, 65] and sum(ref["seq_lens"]) == 494
    assert (ref["batch_size"], ref["max_padding_size"], ref["head_num"], ref["head_size"]) == (8, 128, 12, 64)


@pytest.mark.parametrize("case", PACK["cases"], ids=lambda c: f"B{c['B']}S{c['S']}H{c['H']}D{c['D']}")
def test_oracle_matches_pack_vectors(case):
    B, S, H, D, lens, T = case["B"], case["S"], case["H"], case["D"], case["lens"], case["valid"]
    packed = torch.tensor(case["packed"]).view(1, T, H, D)
    padded = torch.tensor(case["padded"]).view(B, H, S, D)
    assert torch.equal(eager.transpose_pad(packed, B, S, lens, H, D), padded)
    assert torch.equal(eager.transpose_depad(padded, B, T, S, lens, H, D).flatten(), torch.tensor(case["depadded"]))
    valid, off = eager.ft_build_padding_offsets(lens, B, S)
    assert int(valid[0]) == T and off.tolist() == case["offsets"]
    hidden = torch.tensor(case["hidden"]).view(B, S, H * D)
    removed, mask = eager.ft_remove_padding(hidden, off, T, H * D)
    assert removed.flatten().tolist() == case["removed"]
    assert eager.ft_rebuild_padding(removed, mask, T, H * D, B, S).flatten().tolist() == case["rebuilt"]
    assert eager.ft_transpose_remove_padding(torch.tensor(case["transposed_rebuilt"]).view(B, H, S, D), T, B, S, H, D,
                                             mask).flatten().tolist() == case["transposed_removed"]


def test_oracle_matches_math_vectors():
    sm = MATH["softmax"]
    B, H, S = sm["B"], sm["H"], sm["S"]
    got = eager.scale_mask_softmax(B, S, H, torch.tensor(sm["scores"], dtype=torch.float64).view(B, H, S, S),
                                   sm["lens"], acc_dtype=torch.float64)
    assert torch.allclose(got.flatten(), torch.tensor(sm["probs"], dtype=torch.float64), atol=1e-12)
    ln = MATH["layernorm"]
    y, mean, invvar, _ = eager.layer_norm(torch.tensor(ln["x"], dtype=torch.float64).view(ln["n1"], ln["n2"]),
                                          torch.tensor(ln["gamma"], dtype=torch.float64),
                                          torch.tensor(ln["beta"], dtype=torch.float64), ln["eps"],
                                          acc_dtype=torch.float64, out_dtype=torch.float64)
    assert torch.allclose(y.flatten(), torch.tensor(ln["y"], dtype=torch.float64), atol=1e-9)
    assert torch.allclose(mean.double(), torch.tensor(ln["mean"], dtype=torch.float64), atol=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("case", PACK["cases"], ids=lambda c: f"B{c['B']}S{c['S']}H{c['H']}D{c['D']}")
def test_hip_matches_pack_vectors(case, dtype):
    from energonai_amd import kernel as k
    B, S, H, D, lens, T = case["B"], case["S"], case["H"], case["D"], case["lens"], case["valid"]
    print("[case] golden pack", B, S, H, D, dtype, flush=True)
    lens_t = torch.tensor(lens, dtype=torch.int32).cuda()
    packed = torch.tensor(case["packed"]).to(dtype).view(1, T, H, D)
    padded = torch.tensor(case["padded"]).to(dtype).view(B, H, S, D)
    assert torch.equal(k.transpose_pad(packed.cuda(), B, S, lens_t, H, D).cpu(), padded)
    assert torch.equal(k.transpose_depad(padded.cuda(), B, T, S, lens_t, H, D).cpu().flatten(),
                       torch.tensor(case["depadded"]).to(dtype))
    tmp = torch.zeros(B * S, dtype=torch.int32).cuda()
    mask = torch.zeros(B * S, dtype=torch.int32).cuda()
    valid = torch.zeros(1, dtype=torch.int32).cuda()
    k.ft_build_padding_offsets(lens_t, B, S, valid, tmp)
    assert int(valid.item()) == T and tmp[:T].cpu().tolist() == case["offsets"]
    hidden = torch.tensor(case["hidden"]).to(dtype).view(B, S, H * D).cuda()
    removed = k.ft_remove_padding(hidden, tmp, mask, T, H * D)
    assert removed.cpu().flatten().tolist() == case["removed"]
    assert k.ft_rebuild_padding(removed, mask, T, H * D, B, S).cpu().flatten().tolist() == case["rebuilt"]
    buf = torch.full((B, H, S, D), 0.5, dtype=dtype).cuda()
    q = removed.view(T, H, D)
    k.ft_transpose_rebuild_padding(q, q, q, buf, buf.clone(), buf.clone(), B, S, H, D, T, mask)
    assert buf.cpu().flatten().tolist() == case["transposed_rebuilt"]
    assert k.ft_transpose_remove_padding(buf, T, B, S, H, D, mask).cpu().flatten().tolist() == case["transposed_removed"]


@pytest.mark.gpu
def test_hip_matches_math_vectors():
    from energonai_amd import kernel as k
    print("[case] golden math", flush=True)
    sm = MATH["softmax"]
    B, H, S = sm["B"], sm["H"], sm["S"]
    x = torch.tensor(sm["scores"]).view(B, H, S, S).cuda()
    got = k.scale_mask_softmax(B, S, H, x, torch.tensor(sm["lens"], dtype=torch.int32).cuda()).cpu()
    assert torch.allclose(got.flatten().double(), torch.tensor(sm["probs"], dtype=torch.float64), atol=1e-6)
    ln = MATH["layernorm"]
    y, mean, invvar = k.layer_norm_forward(torch.tensor(ln["x"]).view(ln["n1"], ln["n2"]).cuda(),
                                           torch.tensor(ln["gamma"]).cuda(), torch.tensor(ln["beta"]).cuda(),
                                           (ln["n2"],), ln["eps"], return_stats=True)
    assert torch.allclose(y.cpu().flatten().double(), torch.tensor(ln["y"], dtype=torch.float64), atol=1e-5)
    assert torch.allclose(mean.cpu().double(), torch.tensor(ln["mean"], dtype=torch.float64), atol=1e-6)
    assert torch.allclose(invvar.cpu().double(), torch.tensor(ln["invvar"], dtype=torch.float64), rtol=1e-5)
