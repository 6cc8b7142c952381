"""The random numbers of seeded sampling, and what sampling parameters are refused (no GPU)."""
import numpy as np
import pytest

from inferflux_amd.sampling.params import SamplingParams, philox4x32_10, philox_uniform

# Known answers of Philox4x32-10 (the generator's published test vectors: counter, key -> output).
PHILOX_VECTORS = [
    ((0, 0, 0, 0), (0, 0), (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)),
    ((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2, (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)),
    ((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0), (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1)),
]


@pytest.mark.parametrize("counter,key,want", PHILOX_VECTORS)
def test_philox_known_answers(counter, key, want):
    got = philox4x32_10([np.array([w]) for w in counter], [np.array([w]) for w in key])
    assert tuple(int(w[0]) for w in got) == want


def test_uniform_numbers_are_the_top_bits_of_the_first_word():
    """The seed is the key and the count of draws the counter's low 64 bits; 24 bits make the number, so it is below 1."""
    u = philox_uniform(np.array([0, 0xFFFFFFFFFFFFFFFF], dtype=np.uint64), np.array([0, 0xFFFFFFFFFFFFFFFF], dtype=np.uint64))
    assert u.dtype == np.float32
    assert float(u[0]) == (0x6627E8D5 >> 8) / (1 << 24)
    # counter words 2 and 3 are zero for a draw, so the second pair is not the all-ones vector: pin it by its own rounds
    want = philox4x32_10([np.array([0xFFFFFFFF]), np.array([0xFFFFFFFF]), np.array([0]), np.array([0])],
                         [np.array([0xFFFFFFFF]), np.array([0xFFFFFFFF])])
    assert float(u[1]) == (int(want[0][0]) >> 8) / (1 << 24)
    many = philox_uniform(np.full(4096, 7, dtype=np.uint64), np.arange(4096, dtype=np.uint64))
    assert 0.0 <= float(many.min()) and float(many.max()) < 1.0
    assert abs(float(many.mean()) - 0.5) < 0.03 and len(set(many.tolist())) > 4000
    assert philox_uniform(np.array([7]), np.array([5]))[0] == many[5]            # the pair alone decides


@pytest.mark.parametrize("fields", [dict(temperature=-0.1), dict(top_p=0.0), dict(top_p=1.5), dict(top_k=-1), dict(min_p=1.5),
                                    dict(repetition_penalty=0.0), dict(penalty_last_n=-1), dict(max_tokens=0),
                                    dict(logprobs=21), dict(seed=-1), dict(seed=1 << 64)])
def test_parameters_out_of_range_are_refused(fields):
    with pytest.raises(ValueError):
        SamplingParams(**fields).validate()
    SamplingParams().validate()
    SamplingParams(seed=(1 << 64) - 1, temperature=0.7, top_k=5, top_p=0.5, min_p=0.1, logprobs=20).validate()
