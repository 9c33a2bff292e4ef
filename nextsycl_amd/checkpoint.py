"""Conversation checkpoints: a session's KV-cache rows at a position, in host memory and as a file.

The host-side counterpart of the engines' `Checkpoint` and their `save` / `restore` / `copy_session`
(llm/museglimmer/src/engine.rs:223-266, 1334-1375, 1475-1528; llm/qwen35/src/engine.rs:262-302, 2977-3011;
llm/deepseek2/src/engine.rs:243-280, 942-971). The bytes are the reference's, so a file written on either side mounts on
the other:

  buffers  for each cache set in the engine's order, for each of its caches (keys, then values): the rows of the
           positions the cache still reads, [heads][kept(win, pos) .. pos)[row bytes], in position order whatever the
           ring's slot order is
  file     5 bytes of magic ("NSMG1", "NSQ35", "NSDS1", "NSRC1", "NSCK1"), u64 position, u64 buffer count, then per
           buffer u64 length + bytes, all little-endian; GLM's form ("NSCK1") ends with its draft block's state:
           u64 0, or u64 1, u64 a, u64 b, u64 count, count x u32

What differs is how the rows travel. The reference reads one or two runs a head and cache across PCIe, each a waiting
call. Here every cache's rows are put in position order ON the GPU (`ns_attn_kv_rows_copy`, one launch a cache, every
head at once) into one staging buffer, and ONE copy brings the whole checkpoint to the host; `restore` is the same in
reverse, and `copy_session` never leaves the GPU. Nothing here computes on the host: without the HIP library the calls
fail."""
import io
import struct
from collections import namedtuple

import numpy as np

from .core import DevBuf, Error, HostBuf, check

MAGIC = {"museglimmer": b"NSMG1", "qwen35": b"NSQ35", "deepseek2": b"NSDS1", "ricursive": b"NSRC1", "glm5next": b"NSCK1"}

# One layer's caches: `bufs` the device buffers that share a geometry (keys and values; one latent cache for MLA), each
# [heads][cap][row bytes] with position p in slot p % cap; `win` > 0: only the last win - 1 positions are still read.
Ring = namedtuple("Ring", "bufs cap heads win row")


def kept(win, pos):
    """The first position a cache with window `win` still reads at `pos` (llm/museglimmer/src/engine.rs:1358-1361)."""
    return max(0, pos - (win - 1)) if win > 0 else 0


class Checkpoint:
    """A conversation's state at a position, in host memory: `pos`, the buffers (uint8 arrays), their total `bytes`."""

    def __init__(self, pos, bufs, mtp=None):
        self.pos = int(pos)
        self.bufs = [np.frombuffer(b, np.uint8) if not isinstance(b, np.ndarray) else b.view(np.uint8).reshape(-1) for b in bufs]
        self.bytes = sum(b.size for b in self.bufs)
        self.mtp = mtp          # GLM's draft block: (a, b, [next tokens]) or None

    def write_to(self, w, magic=MAGIC["museglimmer"]):
        """The checkpoint as a file (llm/museglimmer/src/engine.rs:230-240; GLM's tail: llm/glm5next/src/engine.rs:527-540)."""
        if len(magic) != 5:
            raise Error("a magic of 5 bytes")
        w.write(magic)
        w.write(struct.pack("<QQ", self.pos, len(self.bufs)))
        for b in self.bufs:
            w.write(struct.pack("<Q", b.size))
            w.write(b.tobytes())
        if magic == MAGIC["glm5next"]:
            if self.mtp is None:
                w.write(struct.pack("<Q", 0))
            else:
                a, b, nxt = self.mtp
                w.write(struct.pack("<QQQQ", 1, a, b, len(nxt)))
                w.write(struct.pack("<%dI" % len(nxt), *nxt))

    @staticmethod
    def read_from(r, magic=MAGIC["museglimmer"]):
        """`write_to`'s file back; another magic or a short file is an Error (llm/museglimmer/src/engine.rs:242-265)."""

        def exact(n):
            b = r.read(n)
            if len(b) != n:
                raise Error("a checkpoint file that ends early")
            return b

        def u():
            return struct.unpack("<Q", exact(8))[0]

        if exact(5) != magic:
            raise Error("not a %s checkpoint" % {v: k for k, v in MAGIC.items()}.get(magic, magic.decode("ascii", "replace")))
        pos, n = u(), u()
        bufs = [np.frombuffer(exact(u()), np.uint8) for _ in range(n)]
        mtp = None
        if magic == MAGIC["glm5next"] and u() == 1:
            a, b, k = u(), u(), u()
            mtp = (a, b, list(struct.unpack("<%dI" % k, exact(4 * k))))
        return Checkpoint(pos, bufs, mtp)

    def to_bytes(self, magic=MAGIC["museglimmer"]):
        w = io.BytesIO()
        self.write_to(w, magic)
        return w.getvalue()


def _align(n):
    return (n + 255) // 256 * 256


def _plan(rings, pos):
    """[(ring, cache, first position, positions, staging offset, bytes)] in the checkpoint's buffer order, staging size."""
    plan, off = [], 0
    for r in rings:
        first = kept(r.win, pos)
        n = pos - first
        if n > r.cap:
            raise Error("%d positions kept in a cache of %d slots" % (n, r.cap))
        for c in r.bufs:
            size = r.heads * n * r.row
            plan.append((r, c, first, n, off, size))
            off = _align(off + size)
    return plan, off


def save(ops, rings, pos):
    """The rows every cache still reads at `pos`, as a Checkpoint (llm/museglimmer/src/engine.rs:1475-1497; a cache
    without a window and `cap` = the session's context is qwen35's and deepseek2's form: llm/qwen35/src/engine.rs:
    2983-2991, llm/deepseek2/src/engine.rs:942-954). One launch a cache, one copy to the host."""
    plan, total = _plan(rings, pos)
    if total == 0:
        return Checkpoint(pos, [np.zeros(0, np.uint8) for _ in plan])
    stage = DevBuf(ops.gpu, total)
    for r, c, first, n, off, size in plan:
        if n > 0:
            ops.kv_rows_copy(c, r.cap, 0, stage.view(off, size), n, first, r.heads, r.row, first, pos)
    g = ops.gpu
    pinned = HostBuf(g, total)
    check(g.api, g.api.copy_from(g.raw, pinned.ptr, stage.ptr, total), "copying a checkpoint from the GPU")
    g.sync()
    host = pinned.array(np.uint8)
    return Checkpoint(pos, [host[off:off + size].copy() for _, _, _, _, off, size in plan])


def restore(ops, rings, max_ctx, ck):
    """A checkpoint's rows back into a session's caches (whose capacities may differ from the saving session's);
    returns the session's new position. Errors as llm/museglimmer/src/engine.rs:1499-1528."""
    if ck.pos > max_ctx:
        raise Error("a checkpoint of %d tokens into a session of %d" % (ck.pos, max_ctx))
    plan, total = _plan(rings, ck.pos)
    if len(ck.bufs) < len(plan):
        raise Error("a short checkpoint")
    for (_, _, _, _, _, size), b in zip(plan, ck.bufs):
        if b.size != size:
            raise Error("a checkpoint of another shape")
    if total == 0:
        return ck.pos
    g = ops.gpu
    pinned = HostBuf(g, total)
    host = pinned.array(np.uint8)
    for (_, _, _, _, off, size), b in zip(plan, ck.bufs):
        host[off:off + size] = b
    stage = DevBuf(g, total)
    check(g.api, g.api.copy_to(g.raw, stage.ptr, pinned.ptr, total), "copying a checkpoint to the GPU")
    for r, c, first, n, off, size in plan:
        if n > 0:
            ops.kv_rows_copy(stage.view(off, size), n, first, c, r.cap, 0, r.heads, r.row, first, ck.pos)
    g.sync()            # the staging buffers are released on return
    return ck.pos


def copy_session(ops, dst_rings, dst_max_ctx, src_rings, src_pos):
    """One session's kept rows into another's caches, GPU to GPU (llm/museglimmer/src/engine.rs:1334-1375); returns the
    destination's new position."""
    if src_pos > dst_max_ctx:
        raise Error("a session of %d tokens into one of %d" % (src_pos, dst_max_ctx))
    for d, s in zip(dst_rings, src_rings):
        first = kept(d.win, src_pos)
        if (d.heads, d.row, len(d.bufs)) != (s.heads, s.row, len(s.bufs)):
            raise Error("sessions of other shapes")
        for dc, sc in zip(d.bufs, s.bufs):
            ops.kv_rows_copy(sc, s.cap, 0, dc, d.cap, 0, d.heads, d.row, first, src_pos)
    return src_pos
