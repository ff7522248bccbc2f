"""GPU parity of the packing helpers against the CPU oracle: byte-for-byte."""
import pytest
import torch

import areal_amd
from oracle import packing as P

pytestmark = pytest.mark.gpu


def _to(d, dev):
    return {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in d.items()}


def _same(a, b):
    assert set(a) == set(b)
    for k in a:
        if torch.is_tensor(a[k]):
            assert a[k].dtype == b[k].dtype and a[k].shape == b[k].shape, k
            assert torch.equal(a[k].cpu(), b[k].cpu()), k
        else:
            assert a[k] == b[k], k


def _batch(lens, S, seed=0):
    g = torch.Generator().manual_seed(seed)
    bs = len(lens)
    am = torch.zeros(bs, S, dtype=torch.bool)
    for i, n in enumerate(lens):
        am[i, :n] = True
    return dict(
        attention_mask=am,
        input_ids=torch.randint(0, 150000, (bs, S), generator=g),
        loss_mask=torch.rand(bs, S, generator=g) < 0.5,
        logprobs=torch.randn(bs, S, generator=g),
        half=torch.randn(bs, S, generator=g).bfloat16(),
        feats3=torch.randn(bs, S, 3, generator=g).bfloat16(),      # 6-byte rows
        feats=torch.randn(bs, S, 5, 8, generator=g),               # 160-byte rows
        bytes3=torch.randint(0, 255, (bs, S, 3), generator=g, dtype=torch.uint8),
        rewards=torch.randn(bs, generator=g),
        tag="x",
    )


@pytest.mark.parametrize("lens,S", [([3, 7, 1, 5], 7), ([1], 1), ([64, 2, 33, 128, 17, 128], 128), ([5, 0, 4], 6)])
def test_pack_tensor_dict(device, lens, S):
    d = _batch(lens, S)
    want = P.pack_tensor_dict(d)
    got = areal_amd.pack_tensor_dict(_to(d, device))
    _same(got, want)


@pytest.mark.parametrize("align", [None, 4, 64])
def test_pad_packed_tensor_dict(device, align):
    g = torch.Generator().manual_seed(3)
    lens = [37, 5, 128, 64, 1, 90]
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    T = sum(lens)
    d = dict(cu_seqlens=cu, max_seqlen=max(lens), input_ids=torch.randint(0, 1000, (T,), generator=g),
             loss_mask=torch.rand(T, generator=g) < 0.5, logprobs=torch.randn(T, generator=g),
             position_ids=torch.cat([torch.arange(n) for n in lens]), other=torch.ones(3), name="mb")
    want, w_pad, w_old, w_align = P.pad_packed_tensor_dict(d, 512, pad_value=0.0, seq_align_to=align)
    got, pad, old, al = areal_amd.pad_packed_tensor_dict(_to(d, device), 512, pad_value=0.0, seq_align_to=align)
    assert (pad, al) == (w_pad, w_align) and torch.equal(old.cpu(), w_old)
    _same(got, want)
    # three-channel position ids
    d["position_ids"] = torch.randint(0, 50, (T, 3), generator=g)
    want, *_ = P.pad_packed_tensor_dict(d, 512, seq_align_to=align)
    got, *_ = areal_amd.pad_packed_tensor_dict(_to(d, device), 512, seq_align_to=align)
    _same(got, want)
    with pytest.raises(ValueError, match="smaller than total length"):
        areal_amd.pad_packed_tensor_dict(_to(d, device), 10)


@pytest.mark.parametrize("V,dtype", [(1000, torch.bfloat16), (151936, torch.bfloat16), (77, torch.float32), (3, torch.bfloat16)])
def test_unpad_logits(device, V, dtype):
    g = torch.Generator().manual_seed(5)
    lens = [13, 5, 31, 2]
    cu = torch.tensor([0, 13, 18, 49, 51], dtype=torch.int32)
    d = dict(cu_seqlens=cu, max_seqlen=31, rows=torch.arange(51))
    padded_d, pad_len, old_cu, _ = P.pad_packed_tensor_dict(d, 64, seq_align_to=8)
    T_pad = padded_d["rows"].shape[0]
    logits = torch.randn(T_pad, V, generator=g).to(dtype)
    want = P.unpad_logits(logits, pad_len, padded_d["cu_seqlens"], old_cu)
    got = areal_amd.unpad_logits(logits.to(device), pad_len, padded_d["cu_seqlens"].to(device), old_cu.to(device))
    assert got.dtype == dtype and torch.equal(got.cpu(), want)
    assert torch.equal(areal_amd.unpad_logits(logits.to(device), pad_len).cpu(), logits[:-pad_len])


def test_pack_full_size_round_trip(device):
    bs, S = 512, 4096
    g = torch.Generator().manual_seed(7)
    lens = torch.randint(1, S + 1, (bs,), generator=g)
    am = (torch.arange(S)[None, :] < lens[:, None]).to(device)
    ids = torch.randint(0, 150000, (bs, S), generator=g).to(device)
    lp = torch.randn(bs, S, generator=g).to(device)
    p = areal_amd.pack_tensor_dict(dict(attention_mask=am, input_ids=ids, logprobs=lp))
    assert p["input_ids"].shape[0] == int(lens.sum()) and p["max_seqlen"] == int(lens.max())
    assert torch.equal(p["input_ids"], ids[am]) and torch.equal(p["logprobs"], lp[am])  # row-major boolean gather


@pytest.mark.parametrize("algorithm,seq_align_to,pad_to_maximum", [("ffd", None, False), ("kk", 64, False),
                                                                  ("ffd", None, True)])
def test_packed_mb_list_matches_oracle_chain(device, algorithm, seq_align_to, pad_to_maximum):
    """Padded batch -> balanced micro-batches -> packed -> page padded (fsdp_engine.py:1778-1786), against the
    oracle's row-by-row split, pack and pad."""
    from areal_amd import microbatch as M
    from oracle import microbatch as OM

    g = torch.Generator().manual_seed(12)
    bs, L = 24, 300
    lens = torch.randint(1, L + 1, (bs,), generator=g)
    attn = (torch.arange(L)[None, :] < lens[:, None]).long()
    data = dict(attention_mask=attn, input_ids=torch.randint(0, 999, (bs, L), generator=g),
                logprobs=torch.randn(bs, L, generator=g), loss_mask=(torch.rand(bs, L, generator=g) < 0.5),
                rewards=torch.randn(bs, generator=g))
    cap = 2048
    spec = M.MicroBatchSpec(n_mbs=2, max_tokens_per_mb=cap, packing_algorithm=algorithm)
    got = M.packed_mb_list({k: v.to(device) for k, v in data.items()}, spec, seq_align_to=seq_align_to,
                           pad_to_maximum=pad_to_maximum)
    ref = M.amend_position_ids(dict(data))
    mbs, group_lens, fwd, bwd = OM.split_padded_tensor_dict(ref, cap, 2, 1, 1, algorithm)
    assert got.group_lens == group_lens and [int(i) for i in got.forward_indices] == fwd
    assert len(got) == len(mbs) >= 2
    for item, mb, n_tok in zip(got, mbs, group_lens):
        packed = P.pack_tensor_dict(mb)
        pad_to = cap if pad_to_maximum else (n_tok + 255) // 256 * 256
        want, pad_len, old_cu, _ = P.pad_packed_tensor_dict(packed, pad_to, 0.0, seq_align_to=seq_align_to)
        assert item.padding_length == pad_len and item.padded_to_length == pad_to
        for key in ("input_ids", "logprobs", "loss_mask", "position_ids", "cu_seqlens"):
            assert torch.equal(item.padded_mb[key].cpu(), want[key]), key
            assert torch.equal(item.orig_mb[key].cpu(), packed[key]), key
        assert int(item.padded_mb["max_seqlen"]) == int(want["max_seqlen"])
        assert torch.equal(item.orig_mb["rewards"].cpu(), data["rewards"])          # not split: shared by every micro-batch
        if seq_align_to is not None:
            assert torch.equal(item.old_cu_seqlens.cpu(), old_cu)
    assert got.max_seqlen == max(int(m["cu_seqlens"][-1]) for m in got.padded_mbs)


def test_unsqueeze_mb_list_adds_the_batch_dimension(device):
    from areal_amd import microbatch as M

    g = torch.Generator().manual_seed(2)
    bs, L = 6, 50
    lens = torch.randint(1, L + 1, (bs,), generator=g)
    attn = (torch.arange(L)[None, :] < lens[:, None]).long()
    data = dict(attention_mask=attn.to(device), input_ids=torch.randint(0, 9, (bs, L), generator=g).to(device),
                rewards=torch.randn(bs, generator=g).to(device))
    mbl = M.unsqueeze_mb_list(M.packed_mb_list(data, M.MicroBatchSpec(n_mbs=2)))
    for item in mbl:
        n = item.padded_to_length
        assert item.padded_mb["input_ids"].shape == (1, n) and item.padded_mb["position_ids"].shape == (1, n)
        assert item.padded_mb["cu_seqlens"].ndim == 1 and item.padded_mb["rewards"].shape == (bs,)
        assert item.orig_mb["input_ids"].ndim == 1                                  # only the padded ones change
    one = M.unsqueeze_packed_tensor_dict(mbl.mbs[0])
    assert one["input_ids"].ndim == 2 and one["input_ids"].shape[0] == 1
