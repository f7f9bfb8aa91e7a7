"""What the model classes of the ragged stack engine share: a checkpoint directory is config.json + model.safetensors (bfloat16
weights carried as uint16 bit patterns, linear weights [out, in]); the class turns its configuration into the engine's flat
key=value description and hands the tensors over.  There is no Python forward pass."""
import os
from typing import Dict

import numpy as np

from .._utils import read_safetensors

PAGE_SIZE = 64


def to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """fp32 array -> bfloat16 bit patterns (uint16), round to nearest even."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16).reshape(a.shape)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << 16).view(np.float32)


class StackModelForCausalLM(object):
    """Subclasses set `architecture` and `config_class` (built from the parsed config.json, with `engine_config()`)."""
    architecture = None
    config_class = None
    page_size = PAGE_SIZE

    def __init__(self, config, tensors: Dict):
        self.config, self.tensors = config, tensors

    @classmethod
    def from_checkpoint(cls, model_dir: str):
        config = cls.config_class.from_json_file(os.path.join(model_dir, 'config.json'))
        return cls(config, read_safetensors(os.path.join(model_dir, 'model.safetensors')))

    def build_stack_engine(self, dtype: str = 'bfloat16', num_blocks: int = 64, num_slots: int = 4, debug_taps: bool = False,
                           build_if_missing: bool = False):
        from ..runtime.stack import StackEngine
        if dtype not in ('bfloat16', 'float32'):
            raise ValueError(f'dtype {dtype!r}: bfloat16 or float32')
        c = self.config.engine_config()
        c.update(dtype=dtype, num_blocks=num_blocks, num_slots=num_slots, debug_taps=int(debug_taps))
        return StackEngine(c, self.tensors, build_if_missing=build_if_missing)
