"""Pins of oracle/packing.py: element-by-element brute force, the properties the reference's own test checks
(tests/test_utils.py:40-75: packed lengths equal the attention-mask sums, unpack + pad restores the batch), and
hand-written tiny cases."""
import torch

from oracle import packing as P


def _batch(lens, S, seed=0):
    g = torch.Generator().manual_seed(seed)
    bs = len(lens)
    am = torch.zeros(bs, S, dtype=torch.bool)
    for i, n in enumerate(lens):
        am[i, :n] = True
    return dict(attention_mask=am, input_ids=torch.randint(0, 1000, (bs, S), generator=g) * am,
                logprobs=torch.randn(bs, S, generator=g) * am, feats=torch.randn(bs, S, 3, generator=g),
                rewards=torch.randn(bs, generator=g), tag="x")


def test_pack_brute_force_and_round_trip():
    lens, S = [3, 7, 1, 5], 7
    d = _batch(lens, S)
    p = P.pack_tensor_dict(d)
    assert p["cu_seqlens"].tolist() == [0, 3, 10, 11, 16] and p["cu_seqlens"].dtype == torch.int32
    assert p["max_seqlen"] == 7 and p["tag"] == "x" and p["rewards"] is d["rewards"] and "attention_mask" not in p
    assert torch.equal(p["cu_seqlens"][1:] - p["cu_seqlens"][:-1], d["attention_mask"].sum(1).int())
    for key in ("input_ids", "logprobs", "feats"):
        flat = [d[key][i, t] for i in range(len(lens)) for t in range(lens[i])]
        assert p[key].shape[0] == sum(lens) and all(torch.equal(a, b) for a, b in zip(p[key], flat))
        back = torch.zeros_like(d[key])
        for i, n in enumerate(lens):
            back[i, :n] = p[key][p["cu_seqlens"][i] : p["cu_seqlens"][i + 1]]
        assert torch.equal(back * d["attention_mask"].reshape(len(lens), S, *[1] * (back.ndim - 2)),
                           d[key] * d["attention_mask"].reshape(len(lens), S, *[1] * (back.ndim - 2)))


def test_pad_packed_hand_case():
    cu = torch.tensor([0, 3, 5], dtype=torch.int32)
    d = dict(cu_seqlens=cu, max_seqlen=3, input_ids=torch.tensor([1, 2, 3, 4, 5]), position_ids=torch.tensor([0, 1, 2, 0, 1]),
             loss_mask=torch.tensor([0, 1, 1, 0, 1]), other=torch.ones(4))
    out, pad_len, old_cu, align = P.pad_packed_tensor_dict(d, 8, pad_value=0)
    assert pad_len == 3 and align is None and torch.equal(old_cu, cu)
    assert out["cu_seqlens"].tolist() == [0, 3, 5, 8] and out["max_seqlen"] == 3
    assert out["input_ids"].tolist() == [1, 2, 3, 4, 5, 0, 0, 0]
    assert out["position_ids"].tolist() == [0, 1, 2, 0, 1, 0, 1, 2] and out["other"] is d["other"]
    # per-sequence alignment to 4: [1 2 3 p][4 5 p p], then page padding to a multiple of lcm(4, 256)
    out, pad_len, old_cu, align = P.pad_packed_tensor_dict(d, 8, pad_value=9, seq_align_to=4)
    assert align == 8 and pad_len == 248 and out["cu_seqlens"].tolist() == [0, 4, 8, 256]
    assert out["input_ids"][:8].tolist() == [1, 2, 3, 9, 4, 5, 9, 9] and out["input_ids"].shape == (256,)
    assert out["position_ids"][:8].tolist() == [0, 1, 2, 3, 0, 1, 2, 3] and out["position_ids"][8:12].tolist() == [0, 1, 2, 3]
    assert out["max_seqlen"] == 248
    # exact fit: nothing to pad
    out, pad_len, _, _ = P.pad_packed_tensor_dict(d, 5)
    assert pad_len == 0 and out is d
    try:
        P.pad_packed_tensor_dict(d, 4)
        assert False
    except ValueError as e:
        assert "smaller than total length" in str(e)


def test_pad_packed_three_channel_position_ids():
    cu = torch.tensor([0, 2, 5], dtype=torch.int32)
    pos = torch.arange(15).reshape(5, 3)
    d = dict(cu_seqlens=cu, max_seqlen=3, position_ids=pos)
    out, _, _, _ = P.pad_packed_tensor_dict(d, 8, seq_align_to=4)
    got = out["position_ids"][:8]
    assert torch.equal(got[:2], pos[:2]) and got[2:4].tolist() == [[0, 0, 0], [1, 1, 1]]
    assert torch.equal(got[4:7], pos[2:5]) and got[7].tolist() == [0, 0, 0]


def test_unpad_logits_inverts_padding():
    g = torch.Generator().manual_seed(1)
    cu = torch.tensor([0, 3, 5, 11], dtype=torch.int32)
    logits = torch.randn(11, 6, generator=g)
    d = dict(cu_seqlens=cu, max_seqlen=6, rows=torch.arange(11))
    out, pad_len, old_cu, _ = P.pad_packed_tensor_dict(d, 16, seq_align_to=4)
    # scatter the logits rows the way the padded batch lays tokens out
    padded = torch.zeros(out["rows"].shape[0], 6)
    new_cu = out["cu_seqlens"]
    for i in range(3):
        n = int(cu[i + 1] - cu[i])
        padded[int(new_cu[i]) : int(new_cu[i]) + n] = logits[int(cu[i]) : int(cu[i + 1])]
    back = P.unpad_logits(padded, pad_len, new_cu, old_cu)
    assert torch.equal(back, logits)
    assert torch.equal(P.unpad_logits(padded, pad_len), padded[:-pad_len])
