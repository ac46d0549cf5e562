"""Writes tests/golden/ref_writer_small.bin with the REFERENCE's own writer
(nncv::rt::MemRefFlatArray::write, compiled into oracle/_ref from /root/reference by
oracle/Makefile).  Run in the build container only: `python tests/golden/make_modelbin_fixture.py`.
The fixture is data (three small seeded tensors in nncv's model.bin byte format)."""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle  # noqa: E402
from nncv_amd import synth  # noqa: E402

tensors = [("conv.weight", synth.normal(1, (2, 3, 3, 3))),
           ("bn.weight", synth.uniform(2, (2,), 0.5, 1.5)),
           ("fc.weight", synth.normal(3, (5, 4)))]
assert oracle.ref_lib() is not None, "oracle/_ref not built"
assert oracle.ref_modelbin_write_f32(os.path.join(HERE, "ref_writer_small.bin"), tensors) == 0
print("wrote", os.path.join(HERE, "ref_writer_small.bin"))
