"""One-step all-to-all: every rank copies chunk j of its input straight to rank j, where it lands at the output
index of the sender.  (The schedule of msccl-tools' examples/mscclang/alltoall_allpairs.py:10-19: automatic
threadblocks, out of place.)"""
from msccl.language import Buffer, chunk


def alltoall_allpairs(size):
    for sender in range(size):
        for receiver in range(size):
            chunk(sender, Buffer.input, receiver).copy(receiver, Buffer.output, sender)
