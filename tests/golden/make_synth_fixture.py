"""Writes tests/golden/synth_seed42.json: the first outputs of the seeded generator
(include/awq_synth.h) computed by the independent numpy statement in tests/helpers.py.
Run from the repository root: python tests/golden/make_synth_fixture.py"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import helpers  # noqa: E402

seed = 42
T_W1 = 2
INPUT = 0x100000
fx = {
    "w1_layer3_packed_first16": helpers.synth_packed(seed, 3, T_W1, 16).tolist(),
    "w1_layer3_scale_first8_bits": helpers.synth_scale(seed, 3, T_W1, 8).view(np.uint16).tolist(),
    "w1_layer3_zp_first8": helpers.synth_zp(seed, 3, T_W1, 8).astype(int).tolist(),
    "normal_first8_bits": helpers.synth_normal(seed, INPUT, 8).astype(np.float16).view(np.uint16).tolist(),
    "tokens_first8": (helpers.synth_hash(seed, INPUT + 1, np.arange(8, dtype=np.uint64)) % np.uint64(151936)).astype(int).tolist(),
}
json.dump(fx, open(os.path.join(HERE, "synth_seed42.json"), "w"), indent=1)
print(fx)
