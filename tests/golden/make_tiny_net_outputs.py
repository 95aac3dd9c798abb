"""Writes tests/golden/tiny_net_outputs.npz: outputs of the CPU oracle (oracle/nn.py) for the seeded
tiny networks of lc0_amd/netgen.py on 8 seeded random-playout positions.

The fixture freezes the whole chain generator -> weight file -> reader -> forward pass, so that a
change in any of them shows up as a diff against numbers that were produced before the change; the
positions are stored as UCI move lists from the start position so that any implementation (a real
lc0 included) can replay them.

  python tests/golden/make_tiny_net_outputs.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from lc0_amd import netgen  # noqa: E402
from oracle import chess as oc  # noqa: E402
from oracle import netread as nr  # noqa: E402
from oracle import nn as onn  # noqa: E402

NETS = ["tiny_resnet", "tiny_resnet_convpolicy", "tiny_attn", "tiny_attn_dense"]
SEED, COUNT = 777, 8


def main():
    pos = oc.random_positions(COUNT, seed=SEED)
    out = {"uci": np.array(pos["uci"]), "masks": pos["masks"], "values": pos["values"]}
    for name in NETS:
        res = onn.BlasNetwork(nr.load(netgen.cached_config(name))).forward(pos["masks"], pos["values"])
        out[name + ".policy"] = res["policy"].astype(np.float32)
        out[name + ".wdl"] = res["wdl"].astype(np.float32)
        out[name + ".m"] = np.asarray(res["m"], np.float32)
    np.savez_compressed(os.path.join(ROOT, "tests", "golden", "tiny_net_outputs.npz"), **out)


if __name__ == "__main__":
    main()
