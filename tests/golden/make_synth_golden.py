"""Writes tests/golden/synth_golden.json: a few values of the seeded generator in
rustingbrain_amd/synth.py, so that a change to the generator (and with it to
every benchmark input) is noticed.  Run from the repository root:

    python tests/golden/make_synth_golden.py
"""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from rustingbrain_amd import synth  # noqa: E402

t = synth.make("c2_decode_d768_e8")
gold = {
    "uniform_seed42_stream7": synth.uniform((6,), 1.0, 42, 7).tolist(),
    "normal_seed42_stream7": synth.normal((6,), 1.0, 42, 7).tolist(),
    "c2_x_first4": t.x[0, :4].tolist(),
    "c2_expert3_down_row5_first4": t.experts[3]["down"][5, :4].tolist(),
}
with open(os.path.join(ROOT, "tests", "golden", "synth_golden.json"), "w") as f:
    json.dump(gold, f, indent=1)
print(gold)
