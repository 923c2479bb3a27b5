"""The engine's host sampler and generator against the plain ones (no GPU)."""
import numpy as np
import pytest

import plain_model as pm
from flambeau_amd.sampling import SamplingParams, Xoshiro256, sample_host


def test_generator_matches_the_plain_one():
    for seed in (0, 1, 42, 2**63 + 5):
        a, b = Xoshiro256(seed), pm.Xoshiro(seed)
        assert [a.next_u64() for _ in range(50)] == [b.next_u64() for _ in range(50)]
        assert [a.next_f32() for _ in range(50)] == [b.next_f32() for _ in range(50)]


@pytest.mark.parametrize("kw", [
    dict(), dict(temperature=0.8), dict(temperature=1.3, top_k=5), dict(temperature=1.0, top_p=0.7),
    dict(temperature=0.9, min_p=0.2), dict(temperature=1.0, top_k=20, top_p=0.9, min_p=0.05),
    dict(temperature=0.0, repetition_penalty=1.8), dict(temperature=0.7, presence_penalty=0.6, frequency_penalty=0.2),
    dict(temperature=0.0, logit_bias={3: 5.0, 400: 1.0}),
])
def test_same_choices_as_the_plain_sampler(kw):
    rng = np.random.default_rng(0)
    history = [int(t) for t in rng.integers(0, 97, 30)]
    ga, gb = Xoshiro256(9), pm.Xoshiro(9)
    same = 0
    for i in range(200):
        logits = (rng.normal(size=97) * 2).astype(np.float32)
        a = sample_host(logits, SamplingParams(**kw), history, ga)
        b = pm.sample(logits, gb, history=history, **kw)
        same += a == b
    assert same >= 198      # the two sum in different orders: a draw on a boundary may differ


def test_parameter_checks():
    with pytest.raises(ValueError):
        SamplingParams(max_tokens=0)
    with pytest.raises(ValueError):
        SamplingParams(top_k=0)
    assert SamplingParams().is_greedy and SamplingParams().device_ok
    # filters (up to 2048 candidates), penalties and a bias of up to 256 entries run on the device
    assert SamplingParams(temperature=1.0, top_p=0.9).device_ok and SamplingParams(temperature=1.0, top_k=2048).device_ok
    assert not SamplingParams(temperature=1.0, top_k=2049).device_ok
    assert SamplingParams(repetition_penalty=1.1).device_ok and SamplingParams(logit_bias={3: 1.0}).device_ok
    assert not SamplingParams(logit_bias={t: 1.0 for t in range(257)}).device_ok
    # a vocabulary beyond what the filtered draw takes sends filters (and only them) to the host sampler
    from flambeau_amd.kernels.library import load
    from flambeau_amd.sampling.params import DEVICE_FILTER_VOCAB_MAX, DEVICE_TOP_K_MAX
    lib = load()
    assert lib.fl_sample_filtered_max_vocab() == DEVICE_FILTER_VOCAB_MAX and lib.fl_sample_filtered_max_k() == DEVICE_TOP_K_MAX
    assert SamplingParams(temperature=1.0, top_p=0.9).device_takes(DEVICE_FILTER_VOCAB_MAX)
    assert not SamplingParams(temperature=1.0, top_p=0.9).device_takes(DEVICE_FILTER_VOCAB_MAX + 1)
    assert SamplingParams(temperature=1.0).device_takes(300000) and SamplingParams(top_k=5).device_takes(300000)   # no filter; greedy
    assert not SamplingParams(temperature=1.0, top_k=3000).device_takes(1000)
    assert SamplingParams(presence_penalty=0.5, frequency_penalty=0.25).penalties == (1.0, 0.5, 0.25)
    assert SamplingParams(temperature=1.0, top_p=0.9).device_filters == (2048, 0.9, 0.0)
    assert SamplingParams(temperature=1.0, top_k=7, min_p=0.1).device_filters == (7, 0.0, 0.1)
    assert SamplingParams(temperature=1.0, top_p=1.0).device_filters == (2048, 0.0, 0.0)
    assert SamplingParams(temperature=1.0).device_filters == (0, 0.0, 0.0)
