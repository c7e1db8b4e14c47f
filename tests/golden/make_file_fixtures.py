#!/usr/bin/env python3
"""Writes the container-format fixtures with the COMPILED REFERENCE (oracle/_ref, built from
/root/reference/src in place): a tiny model saved by the reference's apu_save_dnn_to_file and its
tile graph saved by apu_save_nasm_to_file.  Run here (where the reference is mounted), commit the
outputs; the tests only read them.

    python tests/golden/make_file_fixtures.py
"""
import os
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from aspen_amd import models as M          # noqa: E402
from oracle import ref                     # noqa: E402
from tests import helpers as H             # noqa: E402


def main():
    ref.build()
    cfg, layers, tens, x, batch, seq = H.tiny_case()
    wp = tempfile.mktemp(suffix=".bin")
    M.write_aspen_data(wp, tens)
    net = ref.RefNet(cfg, wp, batch, seq, min_ninst=4, threads=1)
    os.unlink(wp)
    net.save_dnn(os.path.join(HERE, "tiny_ref.aspen"))
    n = net.save_nasm(os.path.join(HERE, "tiny_ref_b2.nasm"), batch, seq, 4)
    net.close()
    print("tiny_ref.aspen", os.path.getsize(os.path.join(HERE, "tiny_ref.aspen")), "bytes;",
          "tiny_ref_b2.nasm", n, "tiles,", os.path.getsize(os.path.join(HERE, "tiny_ref_b2.nasm")), "bytes")


if __name__ == "__main__":
    main()
