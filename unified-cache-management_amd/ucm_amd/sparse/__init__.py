from .hash_encoder import HashEncoder  # noqa: F401
from .decode_step import (GSADecodeStep, GSADecodeStepMLA, SparseDecodeStep,  # noqa: F401
                          SparseDecodeStepMLA)
from .hamming_topk import (cuda_hamming_topk, hamming_score, hamming_topk,  # noqa: F401
                           update_seq_lens)
