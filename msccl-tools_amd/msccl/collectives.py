"""Placeholder for msccl-tools' synthesis-side collective specifications (msccl/collectives.py:
pre/postconditions for the Z3 synthesizer).  Synthesis is not part of this package; the module
exists so that MSCCLang programs that say `from msccl.collectives import *` (as
examples/mscclang/simple/allreduce_ring.py:8 does, without using a name from it) run unchanged.
The collectives MSCCLang programs are written against live in msccl.language.collectives."""
__all__ = []
