"""Host-side behaviour that needs no GPU: config validation, argument errors, the no-fallback rule."""
import pytest
import torch

import areal_amd
from areal_amd import RejectionSamplingConfig, synth


# config validation: the cases of tests/test_rejection_sampling.py:8-41 and :806-839 of the reference
def test_config_validation_messages():
    with pytest.raises(ValueError, match="upper must be > 1.0"):
        RejectionSamplingConfig(metric="ratio", upper=1.0)
    with pytest.raises(ValueError, match="lower must be positive"):
        RejectionSamplingConfig(metric="ratio", lower=-0.1, upper=5.0)
    with pytest.raises(ValueError, match="upper must be positive"):
        RejectionSamplingConfig(metric="kl_k2", upper=0.0)
    with pytest.warns(UserWarning, match="agg=.*is ignored"):
        RejectionSamplingConfig(level="token", agg="max", metric="ratio", upper=5.0)
    with pytest.raises(ValueError, match="action='clamp' only supports metric='ratio'"):
        RejectionSamplingConfig(action="clamp", metric="kl_k2", upper=1.0)
    assert RejectionSamplingConfig(action="clamp", metric="ratio", upper=5.0).lower == 0.0
    with pytest.raises(ValueError, match="lower.*cannot be greater than upper"):
        RejectionSamplingConfig(metric="ratio", lower=3.0, upper=2.0)
    for field in ("level", "action", "metric", "agg"):
        with pytest.raises(ValueError, match=f"{field} must be one of"):
            RejectionSamplingConfig(**{field: "invalid"})
    RejectionSamplingConfig(metric="kl_k1", upper=-0.1)  # k1 may be negative: no positivity rule


def test_argument_errors_come_before_device_work():
    x = torch.randn(2, 4)
    m = torch.ones(2, 4, dtype=torch.bool)
    with pytest.raises(ValueError, match="Invalid importance_sampling_level"):
        areal_amd.ppo_actor_loss_fn(x, x, x, x, 0.2, m, importance_sampling_level="invalid")
    cfg = RejectionSamplingConfig(level="token", metric="ratio", upper=5.0)
    with pytest.raises(ValueError, match="shape"):
        areal_amd.apply_rejection_sampling(torch.zeros(1, 2), torch.zeros(1, 3), torch.ones(1, 2), None, cfg)
    with pytest.raises(ValueError, match="ndim"):
        areal_amd.apply_rejection_sampling(torch.zeros(1, 2, 2), torch.zeros(1, 2, 2), torch.ones(1, 2, 2), None, cfg)


def test_cpu_tensors_are_refused_not_emulated():
    x = torch.randn(4, 16)
    y = torch.zeros(4, dtype=torch.int64)
    with pytest.raises(areal_amd.NativeLibraryError, match="no CPU fallback"):
        areal_amd.gather_logprobs(x, y)
    with pytest.raises(areal_amd.NativeLibraryError, match="no CPU fallback"):
        areal_amd.ppo_actor_loss_fn(x, x, x, x, 0.2, torch.ones(4, 16, dtype=torch.bool))


def test_product_package_does_not_import_the_oracle():
    import pathlib

    pkg = pathlib.Path(areal_amd.__file__).parent
    for py in pkg.rglob("*.py"):
        text = py.read_text()
        assert "import oracle" not in text and "from oracle" not in text, py


def test_synthetic_layouts():
    lengths = synth.lengths_uniform(16, 64, 512, seed=0)
    assert len(lengths) == 16 and all(64 <= n <= 512 for n in lengths)
    cu = synth.cu_from_lengths(lengths)
    assert cu.dtype == torch.int32 and cu[0] == 0 and int(cu[-1]) == sum(lengths)
    mask = synth.prefix_mask(lengths, 0.3)
    for i, n in enumerate(lengths):
        seg = mask[int(cu[i]) : int(cu[i + 1])]
        assert int((~seg).sum()) == int(0.3 * n) and not seg[: int(0.3 * n)].any()
    ln = synth.lengths_lognormal(64, 7.5, 0.6, 128, 4096, seed=0)
    assert all(128 <= n <= 4096 for n in ln)
    assert sum(synth.truncate_to_total(ln, 32768)) == 32768
    adv = synth.grpo_advantages([3] * 32, 16, 0.4, seed=1)
    per_seq = adv[::3]
    for g0 in (0, 16):
        grp = per_seq[g0 : g0 + 16]
        assert abs(float(grp.mean())) < 1e-5  # normalised by the group mean
    alt = synth.alternating_mask([2048], 512)
    assert not alt[:512].any() and alt[512:1024].all() and not alt[1024:1536].any()
    case = synth.config0("cpu", seed=0, V=64, n_seqs=3, lo=4, hi=9)
    assert case.logits.shape == (case.n_tokens, 64) and case.logits.dtype == torch.bfloat16
    assert case.labels.dtype == torch.int64 and case.loss_mask.dtype == torch.bool


def test_synthetic_hidden_state_configurations():
    lengths = synth.lengths_until_total(4, 9, 50, seed=1)
    assert sum(lengths) == 50 and all(1 <= n <= 9 for n in lengths)
    c2 = synth.config2("cpu", seed=0, T=300, H=64, V=640)
    assert c2.hidden.shape == (300, 64) and c2.weight.shape == (640, 64) and c2.logits is None
    assert c2.hidden.dtype == torch.bfloat16 and int(c2.cu_seqlens[-1]) == 300
    assert 0.015 < float(c2.weight.float().std()) < 0.025 and 0.9 < float(c2.hidden.float().std()) < 1.1
    c3 = synth.config3("cpu", seed=0, n_seqs=2, seq_len=2048, H=64, V=128)
    assert c3.ppo["c_clip"] == 3.0 and c3.ppo["eps_clip_higher"] == 0.28
    assert c3.ppo["rejection_sampling"]["upper"] == 5.0
    assert not c3.loss_mask[:512].any() and c3.loss_mask[512:1024].all() and not c3.loss_mask[2048 : 2048 + 512].any()
    c4 = synth.config4("cpu", seed=0, T=400, H=64, V=256, lo=8, hi=32)
    assert c4.temperature == 0.7
    best = (c4.hidden.float() @ c4.weight.float().t()).argmax(-1)
    frac = float((best == c4.labels).float().mean())
    assert 0.12 < frac < 0.30  # 20 % argmax labels (+ chance hits)


def test_infer_token_denominator_cases_of_the_reference():
    """The four cases of tests/test_ppo_stats.py:11-51, inputs and expected shapes transcribed."""
    from areal_amd.engine_glue import infer_token_denominator

    cases = [
        (dict(attention_mask=torch.tensor([[1, 1, 0], [1, 1, 1]]), input_ids=torch.tensor([[11, 12], [13, 14]])),
         torch.zeros(5), (2, 3)),                                               # attention_mask wins
        (dict(input_ids=torch.tensor([[11, 12, 13], [14, 15, 16]])), torch.zeros(2, 3), (2, 3)),   # input_ids
        (dict(input_ids=torch.tensor([11, 12, 13, 0])), torch.zeros(3), (3,)),  # padded tree input_ids: fallback
        (dict(logprobs=torch.zeros(2)), torch.zeros(4), (4,)),                  # no metadata: fallback
        (dict(input_ids=torch.tensor([11, 12]), cu_seqlens=torch.tensor([0, 4], dtype=torch.int32)), torch.zeros(2),
         (4,)),                                                                 # tests/test_ppo_stats.py:54-87
    ]
    for data, fallback, shape in cases:
        n_tokens = infer_token_denominator(data, fallback)
        assert tuple(n_tokens.shape) == shape and n_tokens.dtype == torch.bool and bool(n_tokens.all())


@pytest.mark.parametrize("V,stride,lead", [(50257, 50257, 0), (151936, 151936, 1), (32001, 32004, 5), (64, 64, 0),
                                           (64, 72, 0)])
def test_gradient_array_is_laid_out_like_the_logits(V, stride, lead):
    """The array the fused step writes the gradient into has the row stride of the logits and starts at the same
    offset inside a 16-byte piece of memory (the register kernel's condition for rows that are not on 16-byte
    boundaries); rows do not overlap and nothing is shared with the logits."""
    from areal_amd import functional as F

    T = 5
    flat = torch.zeros(lead + T * stride + 8, dtype=torch.bfloat16)
    while flat.data_ptr() % 16:                      # a base on a 16-byte boundary, whatever the allocator gave
        flat = flat[1:]
    logits = flat.as_strided((T, V), (stride, 1), lead)
    out = F._empty_rows_like(logits, stride)
    assert out.shape == logits.shape and out.dtype == logits.dtype
    assert out.stride(1) == 1 and (out.stride(0) == stride or T == 1)
    assert out.data_ptr() % 16 == logits.data_ptr() % 16 == (2 * lead) % 16
    out.fill_(1.0)
    assert float(flat.abs().sum()) == 0.0
    assert float(out.float().sum()) == T * V
