#!/usr/bin/env python3
"""A few prefill and decode steps of the Pemalorn design at layer sizes of a real model (random weights), for
`rocprofv3 --kernel-trace --stats -- python3 tools/prof_pemalorn.py`: which kernels the time of a step goes to."""
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from hydrainfer_amd.utils import design_bench as db  # noqa: E402

dev = torch.device("cuda:0")
torch.cuda.set_device(dev)
size = db.SIZES[sys.argv[1] if len(sys.argv) > 1 else "w2048"]
model = db._pemalorn(size, torch.bfloat16, dev)
with torch.inference_mode():
    ids, pos, params = db._batch(model, 4, 1024, 1024, torch.bfloat16, dev)
    for _ in range(3):
        model(ids, pos, params)
    ids, pos, params = db._batch(model, 32, 1, 1024, torch.bfloat16, dev)
    for _ in range(10):
        model(ids, pos, params)
torch.cuda.synchronize(dev)
