"""MI355X-native packed-KV decode path of Block-GTQ (gfx950 HIP kernels behind
the reference's Python API)."""
from .allocator import greedy_bit_allocation
from .pipeline import BlockGTQPipeline
from .quantizer import BlockGTQQuantizer

__all__ = ["greedy_bit_allocation", "BlockGTQPipeline", "BlockGTQQuantizer"]
