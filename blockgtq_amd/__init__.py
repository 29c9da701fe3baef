"""MI355X-native packed-KV decode path of Block-GTQ (gfx950 HIP kernels behind
the reference's Python API)."""
from .allocator import greedy_bit_allocation
from .pipeline import BlockGTQPipeline
from .quantizer import BlockGTQQuantizer
from .packed_kv_manager import BlockGTQKVManager
from .production_cache import BlockGTQProductionCache
from .production_decode import production_decode_step, production_prefill
from .fp16_baseline import FP16KVCache, fp16_decode_step
from .calibration import (collect_qk_activations, build_quantizers, bake_q_rotations,
                          save_calibration, load_calibration)
from .prefill import layer_major_prefill

__all__ = [
    "greedy_bit_allocation", "BlockGTQPipeline", "BlockGTQQuantizer",
    "BlockGTQKVManager", "BlockGTQProductionCache",
    "production_decode_step", "production_prefill",
    "FP16KVCache", "fp16_decode_step",
    "collect_qk_activations", "build_quantizers", "bake_q_rotations",
    "save_calibration", "load_calibration",
    "layer_major_prefill",
]
