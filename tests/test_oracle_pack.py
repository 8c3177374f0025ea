"""Pins the oracle's packing functions (CPU only).

Three independent statements of each op must agree: the torch-eager
restatement (oracle/eager.py), the pure-Python replay of the reference CUDA
index arithmetic (oracle/brute.py, tiny inputs) and the plain-C replay
(oracle/kernels_ref.c, medium inputs).  On top of that: the reference test's own
construction on its fixed shape (tests/test_kernel/test_transpose_pad_fusion_kernel.py:6-11,32-47,63-79),
closed forms, inverse pairs and zero padding.
"""
import pytest
import torch

from oracle import brute, cref, eager


def _rand(shape, dtype=torch.float32, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).to(dtype)


TINY = [
    (2, 3, 2, 2, [3, 1]),
    (3, 4, 1, 3, [0, 4, 2]),
    (1, 1, 1, 1, [1]),
    (2, 5, 3, 2, [5, 5]),
]


@pytest.mark.parametrize("B,S,H,D,lens", TINY)
def test_transpose_pad_depad_vs_index_replay(B, S, H, D, lens):
    T = sum(lens)
    src = _rand((1, T, H, D), seed=B + S)
    got = eager.transpose_pad(src, B, S, lens, H, D)
    want = brute.transpose_pad(src.flatten().tolist(), B, S, lens, H, D)
    assert got.flatten().tolist() == want
    back = eager.transpose_depad(got, B, T, S, lens, H, D)
    want_back = brute.transpose_depad(got.flatten().tolist(), B, S, lens, H, D)
    assert back.flatten().tolist() == want_back
    assert torch.equal(back, src)


def test_reference_test_construction(ref_test_shape):
    """The reference test's oracle: permute(0,2,1,3) of the zero-padded tensor, and manual_depad."""
    B, S, H, D, lens = (ref_test_shape[k] for k in ("batch", "seq", "heads", "head_dim", "lens"))
    hidden = torch.zeros(B, S, H * D)
    g = torch.Generator().manual_seed(7)
    for i, n in enumerate(lens):
        hidden[i, :n] = torch.randn(n, H * D, generator=g)
    res_original_pad = hidden.view(B, S, H, D).permute(0, 2, 1, 3)
    # manual_depad
    packed = torch.cat([hidden[i:i + 1, :lens[i]] for i in range(B)], dim=1)
    input_depad = packed.view(1, -1, H, D)
    assert torch.equal(eager.depad(hidden, B, lens), packed)
    assert torch.equal(eager.transpose_pad(input_depad, B, S, lens, H, D), res_original_pad.contiguous())
    assert torch.equal(eager.transpose_depad(res_original_pad.contiguous(), B, sum(lens), S, lens, H, D), input_depad)
    # the C replay of the CUDA kernels says the same, for every storage width
    for dtype in (torch.float32, torch.float16, torch.bfloat16):
        x = input_depad.to(dtype)
        padded = cref.transpose_pad(x, B, S, lens, H, D)
        assert torch.equal(padded, eager.transpose_pad(x, B, S, lens, H, D))
        assert torch.equal(cref.transpose_depad(padded, B, sum(lens), S, lens, H, D), x)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_medium_random_vs_c_replay(seed):
    g = torch.Generator().manual_seed(seed)
    B, S, H, D = 5, 37, 3, 24
    lens = torch.randint(0, S + 1, (B,), generator=g).tolist()
    T = sum(lens)
    src = _rand((1, T, H, D), torch.float16, seed)
    padded = eager.transpose_pad(src, B, S, lens, H, D)
    assert torch.equal(padded, cref.transpose_pad(src, B, S, lens, H, D))
    # padding region is exactly zero
    for b, n in enumerate(lens):
        assert bool((padded[b, :, n:] == 0).all())
    assert torch.equal(eager.transpose_depad(padded, B, T, S, lens, H, D), src)
    # fused QKV width: chunks of the fused result are the three separate results
    fused = _rand((1, T, H, 3 * D), torch.float16, seed + 10)
    out = eager.transpose_pad(fused, B, S, lens, H, 3 * D)
    for part_out, part_in in zip(torch.chunk(out, 3, -1), torch.chunk(fused, 3, -1)):
        assert torch.equal(part_out, eager.transpose_pad(part_in.contiguous(), B, S, lens, H, D))


@pytest.mark.parametrize("B,S,lens", [(3, 4, [2, 0, 4]), (1, 3, [3]), (4, 2, [1, 1, 2, 0])])
def test_offsets_closed_form_vs_serial_kernel(B, S, lens):
    valid, off = eager.ft_build_padding_offsets(lens, B, S)
    t, off_b = brute.build_offsets(lens, B, S)
    assert int(valid[0]) == t == sum(lens)
    assert off.tolist() == off_b
    v_c, off_c = cref.build_offsets(lens, B, S)
    assert int(v_c[0]) == t and off_c.tolist() == off_b
    assert eager.prefix_offsets(lens, B).tolist() == [sum(lens[:i]) for i in range(B + 1)]


def test_offsets_known_answer():
    # lens 2,1 in a bucket of 4: tokens 0,1 have 0 padding rows before them, token 2 has 4-2 = 2
    valid, off = eager.ft_build_padding_offsets([2, 1], 2, 4)
    assert int(valid[0]) == 3 and off.tolist() == [0, 0, 2]


@pytest.mark.parametrize("B,S,H,D,lens", TINY + [(3, 6, 2, 4, [6, 0, 3])])
def test_ft_family(B, S, H, D, lens):
    hid = H * D
    T = sum(lens)
    _, off = eager.ft_build_padding_offsets(lens, B, S)
    src = _rand((B, S, hid), seed=3)
    tgt, mask = eager.ft_remove_padding(src, off, T, hid)
    assert tgt.flatten().tolist() == brute.remove_padding(src.flatten().tolist(), off.tolist(), T, hid)
    assert torch.equal(tgt, eager.depad(src, B, lens))                      # same pack as depad
    c_tgt, c_mask = cref.remove_padding(src, off, T, hid)
    assert torch.equal(c_tgt, tgt) and torch.equal(c_mask, mask)
    rebuilt = eager.ft_rebuild_padding(tgt, mask, T, hid, B, S)
    assert rebuilt.flatten().tolist() == brute.rebuild_padding(tgt.flatten().tolist(), mask.tolist(), T, hid, B * S)
    assert torch.equal(rebuilt, cref.rebuild_padding(tgt, mask, T, hid, B, S))
    for b, n in enumerate(lens):                                            # inverse on valid rows, zero elsewhere
        assert torch.equal(rebuilt[b, :n], src[b, :n])
        assert bool((rebuilt[b, n:] == 0).all())
    q = tgt.view(T, H, D)
    buf = torch.full((B, H, S, D), 9.0)
    eager.ft_transpose_rebuild_padding(q, q, q, buf, buf.clone(), buf.clone(), B, S, H, D, T, mask)
    ref_buf = [9.0] * (B * H * S * D)
    brute.transpose_rebuild_padding(q.flatten().tolist(), ref_buf, S, H, D, mask.tolist(), T)
    assert buf.flatten().tolist() == ref_buf
    c_buf = torch.full((B, H, S, D), 9.0)
    cref.transpose_rebuild_padding(q, c_buf, S, H, D, mask, T)
    assert torch.equal(c_buf, buf)
    padded = eager.transpose_pad(q.reshape(1, T, H, D), B, S, lens, H, D)
    for b, n in enumerate(lens):                                            # agrees with transpose_pad on valid rows
        assert torch.equal(buf[b, :, :n], padded[b, :, :n])
        assert bool((buf[b, :, n:] == 9.0).all())                           # padding untouched
    removed = eager.ft_transpose_remove_padding(buf, T, B, S, H, D, mask)
    assert removed.flatten().tolist() == brute.transpose_remove_padding(buf.flatten().tolist(), S, H, D,
                                                                         mask.tolist(), T)
    assert torch.equal(removed, cref.transpose_remove_padding(buf, S, H, D, mask, T))
    assert torch.equal(removed, eager.transpose_depad(padded, B, T, S, lens, H, D).reshape(1, T, hid))


def test_depad_left_padding_is_the_flip():
    B, S, hid = 3, 6, 5
    lens = [6, 2, 4]
    src = _rand((B, S, hid), seed=5)
    left = eager.depad(src, B, lens, left_padded=True)
    flipped = eager.depad(torch.flip(src, dims=[1]), B, lens)
    # flipping the sequence axis turns left padding into right padding and reverses each sequence
    t = 0
    for n in lens:
        assert torch.equal(left[0, t:t + n], torch.flip(flipped[0, t:t + n], dims=[0]))
        t += n
