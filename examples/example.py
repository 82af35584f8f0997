#!/usr/bin/env python3
"""The call sequence of the reference's example (/root/reference/example.py:20-33) on the
MI355X sampler: B=4 rows of V=131072 uniform logits, temperature 1, top_p 0.5, then the same
with presence / repetition penalties carried over three decode steps.

    python examples/example.py
"""
import os
import sys

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))

import torch

import rapid_sampling_amd as sample

batch_size, vocab_size = 4, 131072
temperature, top_p, top_k = 1.0, 0.5, -1
presence_penalty, repetition_penalty, penalty_decay = 1.0, 0.1, 0.996

states = sample.setup_rand(0, batch_size)
logits = torch.rand(batch_size, vocab_size).to(0)
penalties = torch.zeros(batch_size, vocab_size).to(0)
print(logits.shape)

samples = sample.batch_sampling_temperature_topk_topp(logits, states, temperature, top_k, top_p)
print("plain:", samples.tolist())

for step in range(3):
    samples = sample.batch_sampling_repetition_temperature_topk_topp(
        logits, penalties, states, presence_penalty, repetition_penalty, penalty_decay,
        temperature, top_k, top_p)
    print("with penalties, step %d:" % step, samples.tolist(),
          "penalised tokens per row:", (penalties != 0).sum(dim=1).tolist())
