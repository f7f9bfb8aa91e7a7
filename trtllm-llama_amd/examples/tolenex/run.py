#!/usr/bin/env python3
"""Greedy generation with a Tolenex checkpoint (config.json + model.safetensors) on the ragged stack engine - the counterpart of
examples/llama_quant/run.py for models that are served straight from a checkpoint directory:

    python run.py --model_dir DIR --input_tokens prompt.csv|prompt.npy --max_output_len 32 [--dtype bfloat16|float32]

--input_tokens: one prompt per CSV row (or a 1-D / 2-D .npy); several prompts run as one continuously batched job.  There is
no tokenizer for this design: ids in, ids out (--output_csv / --output_npy, prompt followed by the generated tokens)."""
import argparse
import csv
import os
import sys
import time

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), '..', '..'))

from tensorrt_llm.models import load_model  # noqa: E402
from tensorrt_llm.runtime import RaggedGenerationSession, SamplingConfig  # noqa: E402


def parse_arguments(args=None):
    p = argparse.ArgumentParser()
    p.add_argument('--model_dir', type=str, required=True)
    p.add_argument('--max_output_len', type=int, required=True)
    p.add_argument('--dtype', type=str, default='bfloat16', choices=['bfloat16', 'float32'])
    p.add_argument('--input_tokens', dest='input_file', type=str, required=True,
                   help='CSV (one prompt per row) or Numpy file with token ids')
    p.add_argument('--end_id', type=int, default=-1, help='token that ends a request (default: none)')
    p.add_argument('--pad_id', type=int, default=0)
    p.add_argument('--max_sequences', type=int, default=4, help='requests that are live at once (state slots)')
    p.add_argument('--max_batch_tokens', type=int, default=2048, help='tokens per step (prompts are cut to fit)')
    p.add_argument('--output_csv', type=str, default=None)
    p.add_argument('--output_npy', type=str, default=None)
    return p.parse_args(args)


def read_prompts(path):
    if path.endswith('.csv'):
        with open(path) as f:
            return [[int(v) for v in row] for row in csv.reader(f) if row]
    a = np.load(path)
    return [a.astype(np.int64).tolist()] if a.ndim == 1 else [r.tolist() for r in a]


def generate(model_dir, max_output_len, dtype='bfloat16', input_file=None, end_id=-1, pad_id=0, max_sequences=4,
             max_batch_tokens=2048, output_csv=None, output_npy=None):
    prompts = read_prompts(input_file)
    model = load_model(model_dir)
    page = model.page_size
    live = sorted((len(p) + max_output_len for p in prompts), reverse=True)[:max_sequences]
    session = RaggedGenerationSession(model, dtype=dtype, max_tokens=sum(-(-n // page) * page for n in live),
                                      max_sequences=max_sequences, max_batch_tokens=max_batch_tokens, build_if_missing=True)
    t0 = time.time()
    outs = session.decode_batch(prompts, SamplingConfig(end_id=end_id, pad_id=pad_id), max_output_len)
    dt = time.time() - t0
    rows = [list(p) + o.tolist() for p, o in zip(prompts, outs)]
    if output_csv:
        with open(output_csv, 'w') as f:
            csv.writer(f).writerows(rows)
    if output_npy:
        width = max(len(r) for r in rows)
        np.save(output_npy, np.array([r + [pad_id] * (width - len(r)) for r in rows], np.int32))
    for r, p in zip(rows, prompts):
        print('Output ids:', r[len(p):])
    print(f'{model.architecture.lower()}-run ({sum(len(o) for o in outs)} tokens in {dt:.3f} sec)')
    return rows


if __name__ == '__main__':
    generate(**vars(parse_arguments()))
