"""ctypes binding of include/tllm_stack_api.h: the ragged-batch step executor for decoder stacks described at run time.

`StackEngine` owns a tllm_stack_t.  It is the compute half only - which page and which state slot a sequence uses is the
business of the cache managers in kv_cache_manager.py, and what a step contains that of the scheduler (scheduler.py) or of a
caller that drives `RaggedGenerationSession.step` itself."""
import ctypes
import os
import subprocess
from typing import Dict, Optional, Sequence

import numpy as np

_LIB_NAME = 'libtllm_stack_engine.so'
FLOAT, BF16 = 0, 7  # nvinfer1::DataType codes

_lib = None


def lib_path() -> str:
    return os.path.join(os.path.dirname(os.path.dirname(os.path.realpath(__file__))), 'libs', _LIB_NAME)


def build_library(jobs: Optional[int] = None):
    """`make stack` in csrc: compiles the engine and the kernels it launches, nothing of the other libraries."""
    csrc = os.path.join(os.path.dirname(os.path.dirname(os.path.dirname(os.path.realpath(__file__)))), 'csrc')
    jobs = jobs or min(16, os.cpu_count() or 1)
    subprocess.run(['make', '-C', csrc, 'stack', '-j', str(jobs)], check=True, stdout=subprocess.DEVNULL)


class Batch(ctypes.Structure):
    _fields_ = [('n_tokens', ctypes.c_int32), ('n_entries', ctypes.c_int32), ('n_want', ctypes.c_int32),
                ('max_blocks', ctypes.c_int32), ('tokens', ctypes.c_void_p), ('ent_count', ctypes.c_void_p),
                ('ent_pos0', ctypes.c_void_p), ('ent_slot', ctypes.c_void_p), ('block_table', ctypes.c_void_p),
                ('want_rows', ctypes.c_void_p)]


def load_library(build_if_missing: bool = False):
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not os.path.exists(path):
        if not build_if_missing:
            raise RuntimeError(f'{path} not found: build it with `make -C trtllm-llama_amd/csrc stack` '
                               f'(or __graft_entry__.build()); there is no CPU fallback')
        build_library()
    lib = ctypes.CDLL(path)
    c = ctypes
    lib.tllm_last_error.restype = c.c_char_p
    lib.tllm_stack_create.argtypes = [c.c_char_p]
    lib.tllm_stack_create.restype = c.c_void_p
    lib.tllm_stack_set_tensor.argtypes = [c.c_void_p, c.c_char_p, c.c_int32, c.POINTER(c.c_int64), c.c_int32, c.c_void_p]
    lib.tllm_stack_set_tensor.restype = c.c_int32
    lib.tllm_stack_finalize.argtypes = [c.c_void_p]
    lib.tllm_stack_finalize.restype = c.c_int32
    lib.tllm_stack_step.argtypes = [c.c_void_p, c.POINTER(Batch), c.c_void_p, c.c_void_p, c.c_void_p]
    lib.tllm_stack_step.restype = c.c_int32
    for name in ('page_size', 'num_blocks', 'num_slots', 'vocab', 'layer_runs'):
        f = getattr(lib, 'tllm_stack_' + name)
        f.argtypes = [c.c_void_p]
        f.restype = c.c_int32
    lib.tllm_stack_weight_bytes.argtypes = [c.c_void_p]
    lib.tllm_stack_weight_bytes.restype = c.c_int64
    lib.tllm_stack_step_bytes.argtypes = [c.c_void_p, c.c_int32, c.c_int64, c.c_int32]
    lib.tllm_stack_step_bytes.restype = c.c_int64
    lib.tllm_stack_get_tap.argtypes = [c.c_void_p, c.c_int32, c.c_void_p, c.c_size_t]
    lib.tllm_stack_get_tap.restype = c.c_int32
    lib.tllm_stack_destroy.argtypes = [c.c_void_p]
    lib.tllm_stack_destroy.restype = None
    _lib = lib
    return lib


def last_error() -> str:
    return load_library().tllm_last_error().decode('utf-8', 'replace')


class StackEngine:
    """config: flat dict of the keys include/tllm_stack_api.h lists; tensors: name -> (numpy array, 'float32' | 'bfloat16')
    where a bfloat16 tensor is carried as uint16 bit patterns."""

    def __init__(self, config: Dict, tensors: Dict, build_if_missing: bool = False):
        lib = load_library(build_if_missing)
        text = '\n'.join(f'{k}={v}' for k, v in config.items())
        self._h = lib.tllm_stack_create(text.encode())
        if not self._h:
            raise RuntimeError(f'tllm_stack_create failed: {last_error()}')
        for name, (a, kind) in tensors.items():
            a = np.ascontiguousarray(a)
            if kind == 'bfloat16':
                assert a.dtype == np.uint16, name
                code = BF16
            else:
                a = a.astype(np.float32, copy=False)
                code = FLOAT
            dims = (ctypes.c_int64 * max(a.ndim, 1))(*a.shape)
            if lib.tllm_stack_set_tensor(self._h, name.encode(), code, dims, a.ndim, a.ctypes.data):
                raise RuntimeError(f'set_tensor({name}) failed: {last_error()}')
        if lib.tllm_stack_finalize(self._h):
            err = last_error()
            self.close()
            raise RuntimeError(f'tllm_stack_finalize failed: {err}')
        self.page_size = lib.tllm_stack_page_size(self._h)
        self.num_blocks = lib.tllm_stack_num_blocks(self._h)
        self.num_slots = lib.tllm_stack_num_slots(self._h)
        self.vocab = lib.tllm_stack_vocab(self._h)
        self.layer_runs = lib.tllm_stack_layer_runs(self._h)
        self.width = int(config['width'])
        self._last_tokens = 0

    @staticmethod
    def _i32(a) -> np.ndarray:
        return np.ascontiguousarray(np.asarray(a), dtype=np.int32)

    def step(self, tokens: Sequence[int], counts: Sequence[int], pos0: Sequence[int], slots: Sequence[int], block_table,
             want_rows: Sequence[int], return_logits: bool = True, stream: int = 0):
        """One packed step.  block_table: int32 [entries, max_blocks].  Returns (logits fp32 [n_want, vocab] or None,
        next ids int32 [n_want]): the arg-max of every wanted row is the greedy sampler's choice."""
        tokens, counts, pos0, slots = self._i32(tokens), self._i32(counts), self._i32(pos0), self._i32(slots)
        table, want = self._i32(block_table), self._i32(want_rows)
        assert table.ndim == 2 and table.shape[0] == len(counts) == len(pos0) == len(slots)
        b = Batch(len(tokens), len(counts), len(want), table.shape[1], tokens.ctypes.data, counts.ctypes.data, pos0.ctypes.data,
                  slots.ctypes.data, table.ctypes.data, want.ctypes.data if len(want) else None)
        logits = np.empty((len(want), self.vocab), np.float32) if (return_logits and len(want)) else None
        ids = np.empty(len(want), np.int32)
        rc = load_library().tllm_stack_step(self._h, ctypes.byref(b), logits.ctypes.data if logits is not None else None,
                                            ids.ctypes.data if len(want) else None, stream)
        if rc:
            raise RuntimeError(f'tllm_stack_step failed: {last_error()}')
        self._last_tokens = len(tokens)
        return logits, ids

    def tap(self, run: int) -> np.ndarray:
        """debug_taps=1: the residual stream behind layer run `run` of the last step, fp32 [tokens, width]."""
        out = np.empty((self._last_tokens, self.width), np.float32)
        if load_library().tllm_stack_get_tap(self._h, run, out.ctypes.data, out.size):
            raise RuntimeError(f'tllm_stack_get_tap failed: {last_error()}')
        return out

    def weight_bytes(self) -> int:
        return int(load_library().tllm_stack_weight_bytes(self._h))

    def step_bytes(self, n_tokens: int, context_tokens: int, n_entries: int) -> int:
        return int(load_library().tllm_stack_step_bytes(self._h, n_tokens, context_tokens, n_entries))

    def close(self):
        if getattr(self, '_h', None):
            load_library().tllm_stack_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
