"""Host side of sampling (no GPU): options, the random stream and the device records."""
import struct

import pytest

import plain_gpt2 as P
from deliverance_amd.sampling import GeneratorParameters, JavaRandom, device_record, top_k_candidate_count


def test_defaults_are_the_reference_defaults():
    p = GeneratorParameters()
    # core/src/main/java/io/teknek/deliverance/generator/GeneratorParameters.java:12-28
    assert p.temperature == 0.0 and p.seed == 42 and p.ntokens is None and p.max_tokens is None
    assert p.top_k is None and p.top_p is None and p.uniform_top_p is None and p.xtc_threshold is None
    q = p.with_temperature(0.8).with_top_k(40).with_top_p(0.9).with_seed(7).with_max_tokens(5).with_ntokens(50)
    assert (q.temperature, q.top_k, q.top_p, q.seed, q.max_tokens, q.ntokens) == (0.8, 40.0, 0.9, 7, 5, 50)
    assert p.temperature == 0.0                      # the setters return a new record


@pytest.mark.parametrize("kw", [dict(temperature=-1), dict(top_k=0), dict(top_p=0.0), dict(top_p=1.2),
                                dict(uniform_top_p=0.5), dict(uniform_top_p=0.5, top_p=0.9),
                                dict(temperature=0.7, top_k=5, xtc_threshold=0.1), dict(max_tokens=0)])
def test_bad_options_are_refused(kw):
    with pytest.raises(ValueError):
        GeneratorParameters(**kw).validate()


def test_random_stream_is_javas():
    a, b = JavaRandom(42), P.JavaRandom(42)
    xs = [a.next_float() for _ in range(5)]
    assert xs == [b.next_float() for _ in range(5)]
    assert abs(xs[0] - 0.7275637) < 1e-6 and all(0 <= x < 1 for x in xs)
    assert JavaRandom(1).next_float() != JavaRandom(2).next_float()


def test_top_k_counts():
    # core/src/test/java/io/teknek/deliverance/model/TopKSamplerTest.java:13-21
    assert top_k_candidate_count(64.0, 262144) == 64
    assert top_k_candidate_count(0.10, 100) == 90
    assert top_k_candidate_count(5000.0, 100) == 100
    with pytest.raises(ValueError):
        top_k_candidate_count(0.0, 100)


def test_records_draw_in_the_reference_order():
    def fields(p, rng):
        return struct.unpack("<fififfii", device_record(p, rng, 1000))
    # greedy: one draw (made with the sampler, unused)
    r = JavaRandom(42); ref = JavaRandom(42)
    f = fields(GeneratorParameters(), r)
    ref.next_float()
    assert f[0] == 0.0 and f[4] == 0.0 and r.next_float() == ref.next_float()
    # temperature: the second draw is the pick
    r = JavaRandom(42); ref = JavaRandom(42)
    f = fields(GeneratorParameters(temperature=0.8, top_k=50, top_p=0.9), r)
    ref.next_float(); u = ref.next_float()
    assert f[0] == pytest.approx(0.8) and f[1] == 50 and f[2] == pytest.approx(0.9) and f[3] == 0
    assert f[4] == pytest.approx(u) and r.next_float() == ref.next_float()
    # xtc with temperature: two pickers draw, the second decides
    r = JavaRandom(42); ref = JavaRandom(42)
    f = fields(GeneratorParameters(temperature=0.8, xtc_threshold=0.1, xtc_probability=0.5), r)
    ref.next_float(); ref.next_float(); d = ref.next_float()
    assert f[5] == pytest.approx(0.1) and f[6] == int(not d > 0.5) and r.next_float() == ref.next_float()


def test_the_reference_default_nucleus_is_an_explicit_option_here():
    """The reference sets top_p = 0.10 when the temperature is positive and no filter is given
    (core/src/main/java/io/teknek/deliverance/model/AbstractGeneratorSampler.java:107-110); here no
    filter means none.  On the reference's own test logits (TopKSamplerTest.java:23-54: 5, 4, 3, 2, 1;
    softmax 0.636, 0.234, 0.086, 0.032, 0.012) a nucleus of 0.10 holds the first token alone, so with
    ``top_p=0.1`` every draw gives token 0, as the reference's default does; without a filter the draw
    walks the whole softmax."""
    import numpy as np
    logits = np.array([5.0, 4.0, 3.0, 2.0, 1.0])
    cdf = np.cumsum(np.exp(logits - 5.0) / np.exp(logits - 5.0).sum())
    for u in (0.0, 0.3, 0.64, 0.9, 0.999999):
        assert P.sample_top_k_top_p(logits, 1.0, None, 0.10, None, u) == 0
        assert P.sample_top_k_top_p(logits, 1.0, None, None, None, u) == int(np.searchsorted(cdf, u, side="right"))
    # the record that goes to the device carries exactly what was asked for: no silent nucleus
    fields = struct.unpack("<fififfii", device_record(GeneratorParameters(temperature=1.0), JavaRandom(1), 5))
    assert fields[1] == 0 and fields[2] == 0.0
    fields = struct.unpack("<fififfii", device_record(GeneratorParameters(temperature=1.0, top_p=0.1), JavaRandom(1), 5))
    assert fields[2] == pytest.approx(0.1)
