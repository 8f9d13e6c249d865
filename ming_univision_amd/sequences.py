"""Cache-sequence bookkeeping shared by the decoders' callers.

A decoder owns arenas indexed by a cache-sequence number (`BailingMoeDecoder.kv_cache[:, seq]`, `PizitarDecoder.latent[a][seq]`);
`SequenceSlots` hands those numbers out and takes them back, lowest free number first, and grows the decoder's arenas through its
`ensure_sequences` when every number is taken.  A number that is given back is reused by the next request: nothing is cleared,
because a sequence's length — kept here — bounds what any kernel reads of it.

`rows_of_spans` turns the pieces of sequences that one pass through a stack holds into the per-row int32 arrays the step
functions read.
"""
import numpy as np


class SequenceSlots:
    def __init__(self, decoder, first=0):
        self.dec = decoder
        self.first = first                  # numbers below belong to someone else (e.g. a multi-round conversation)
        self.free = []                      # returned numbers
        self.next = first                   # lowest number never handed out
        self.length = {}                    # live sequence -> tokens it holds

    def alloc(self):
        if self.free:
            seq = min(self.free)
            self.free.remove(seq)
        else:
            seq = self.next
            self.next += 1
            self.dec.ensure_sequences(seq + 1)
        self.length[seq] = 0
        return seq

    def release(self, seq):
        if seq not in self.length:
            raise KeyError(f"cache sequence {seq} is not live")
        del self.length[seq]
        self.free.append(seq)

    def live_tokens(self):
        return sum(self.length.values())


def rows_of_spans(spans, block_rows, chunk_rows=0):
    """spans: [(seq, n rows, past)] in row order -> dict of int32 numpy arrays: row_seq, row_slot (= position), row_back (earlier
    rows of the same sequence in this pass), row_len (= slot + 1), blk_tab [n_blk, 2] (first row, rows <= block_rows; a block never
    crosses a span), and max_len.  chunk_rows > 0: also chunk_tab [n_chunks, 2], the same cut in pieces of <= chunk_rows rows (the
    chunks of a recurrence's scan)."""
    seqs, slots, backs, blks, chunks = [], [], [], [], []
    r0 = 0
    for seq, n, past in spans:
        seqs.append(np.full(n, seq, np.int32))
        slots.append(np.arange(past, past + n, dtype=np.int32))
        backs.append(np.arange(n, dtype=np.int32))
        b0 = np.arange(0, n, block_rows, dtype=np.int32)
        blks.append(np.stack([r0 + b0, np.minimum(block_rows, n - b0)], 1))
        if chunk_rows > 0:
            c0 = np.arange(0, n, chunk_rows, dtype=np.int32)
            chunks.append(np.stack([r0 + c0, np.minimum(chunk_rows, n - c0)], 1))
        r0 += n
    slot = np.concatenate(slots)
    out = dict(row_seq=np.concatenate(seqs), row_slot=slot, row_back=np.concatenate(backs), row_len=slot + 1,
               blk_tab=np.ascontiguousarray(np.concatenate(blks).astype(np.int32)), max_len=int(slot.max()) + 1)
    if chunk_rows > 0:
        out["chunk_tab"] = np.ascontiguousarray(np.concatenate(chunks).astype(np.int32))
    return out
