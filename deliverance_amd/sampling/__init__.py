from .params import GeneratorParameters
from .sampler import JavaRandom, device_record, greedy_record, top_k_candidate_count, RECORD_WORDS

__all__ = ["GeneratorParameters", "JavaRandom", "device_record", "greedy_record",
           "top_k_candidate_count", "RECORD_WORDS"]
