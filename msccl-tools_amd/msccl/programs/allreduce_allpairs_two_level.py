"""Two-level all-pairs all-reduce: the all-pairs exchange of msccl-tools' msccl/programs/allreduce_allpairs.py:6-28
used twice, inside groups and across them -- the split of examples/mscclang/hierarchical_allreduce.py:13-77 with
every ring of that program replaced by a one-step exchange.  Seven moving steps deep for any number of ranks, against
the 2(local + groups) - 1 hand-offs of the ring-based two-level program."""
from msccl.language import Buffer, chunk


def allreduce_allpairs_two_level(num_groups, group_size):
    """AllReduce(G*L, G*L, inplace) over G groups of L ranks; rank (g, l) = g*L + l; chunk b*G + s lies in block b (owned, inside
    every group, by local rank b) and is sub-block s of it (owned, among the ranks with local index b, by group s).
      1. inside a group every rank sends block b to local rank b's scratch, which folds the copies in (own value first,
         then peers ascending): rank (g, l) holds the group's sum of block l;
      2. across groups rank (g, l) sends sub-block s of block l to rank (s, l)'s scratch, which folds them in: rank (g, l)
         holds the total of chunk l*G + g;
      3. that chunk goes back to every rank (g', l): block l is complete on all ranks with local index l;
      4. block l goes to every rank of the group.
    Threadblock l' of a rank talks to local peer l' (both ways), threadblock L + g' to the peer in group g'; the folds of
    step 1 are spread over the first G threadblocks by sub-block, the fold of step 2 is threadblock L + g's."""
    G, L = num_groups, group_size
    rank = lambda g, l: g * L + l
    for g in range(G):                      # 1. reduce-scatter inside the groups
        for src in range(L):
            for dst in range(L):
                if src != dst:
                    chunk(rank(g, src), Buffer.input, dst * G, size=G).copy(rank(g, dst), "inside", sendtb=dst, recvtb=src)
    for g in range(G):
        for l in range(L):
            for k in range(G * (L - 1)):
                chunk(rank(g, l), Buffer.input, l * G + k % G).reduce(chunk(rank(g, l), "inside", k), sendtb=k % G)
    for l in range(L):                      # 2. reduce-scatter across the groups
        for src in range(G):
            for dst in range(G):
                if src != dst:
                    chunk(rank(src, l), Buffer.input, l * G + dst).copy(rank(dst, l), "across", sendtb=L + dst, recvtb=L + src)
    for l in range(L):
        for g in range(G):
            for k in range(G - 1):
                chunk(rank(g, l), Buffer.input, l * G + g).reduce(chunk(rank(g, l), "across", k), sendtb=L + g)
    for l in range(L):                      # 3. all-gather across the groups
        for src in range(G):
            for dst in range(G):
                if src != dst:
                    chunk(rank(src, l), Buffer.input, l * G + src).copy(rank(dst, l), Buffer.input, l * G + src, sendtb=L + dst, recvtb=L + src)
    for g in range(G):                      # 4. all-gather inside the groups
        for src in range(L):
            for dst in range(L):
                if src != dst:
                    chunk(rank(g, src), Buffer.input, src * G, size=G).copy(rank(g, dst), Buffer.input, src * G, sendtb=dst, recvtb=src)
