"""Canary blocks in the C heap of the test process.

Three runs of the GPU suite found small heap buffers of the *test process* changed behind their owner's
back: 8-byte words at offset 8 of former 16-byte-aligned allocations, each lower by exactly 6, inside a
920-byte numpy buffer that had just been allocated — every time the first small allocations made after an
encoder-stack handle with a captured HIP graph had been destroyed.  That is what references dropped
through dangling pointers into freed-and-recycled blocks look like (a reference count sits at offset 8 of
such an object, behind its vtable pointer).  Nothing in this library's host code counts references that
way (its only shared_ptr control block outlives every copy, and the host code is clean under
AddressSanitizer), so the writer is taken to be another component of the process.

This module does two things about it.  It *absorbs*: after every test it takes the heap blocks that have
just been freed — several of every small size class, straight from malloc — fills them with a known byte
and holds them until the test after next, so a late write through a dangling pointer lands in a canary and
not in the next test's arrays.  And it *reports*: every held block is compared with its fill when it is
let go; a changed word is written down (block size, offset, old and new value, their difference, the
test that had just ended) in ``report()`` and, when the environment variable ET_CANARY_REPORT names a
file, appended to that file; the test session prints the list at its end.  A hit does not fail
a test by itself: what the library is given is protected separately (tests/harness.py generates every
index structure twice and compares digests at every hand-over)."""
from __future__ import annotations

import ctypes
import os

_libc = ctypes.CDLL(None)
_libc.malloc.restype = ctypes.c_void_p
_libc.malloc.argtypes = [ctypes.c_size_t]
_libc.free.argtypes = [ctypes.c_void_p]

FILL = 0xA5
SIZES = tuple(range(24, 1048, 16)) + (1536, 2048, 3072, 4096)  # usable sizes of the small malloc bins
PER_SIZE = 9  # a thread cache holds at most 7 freed blocks of a size

_generations: list = []  # [(label, [(address, size), ...]), ...], oldest first
_hits: list = []


def take(label: str) -> None:
    """Grab freshly freed small blocks and fill them; `label` names what has just ended."""
    blocks = []
    for size in SIZES:
        for _ in range(PER_SIZE):
            p = _libc.malloc(size)
            if p:
                ctypes.memset(p, FILL, size)
                blocks.append((p, size))
    _generations.append((label, blocks))


def _check(label: str, blocks, when: str) -> None:
    want8 = bytes([FILL]) * 8
    for p, size in blocks:
        raw = ctypes.string_at(p, size)
        if raw.count(FILL) == size:
            continue
        for off in range(0, size - size % 8, 8):
            got = raw[off:off + 8]
            if got != want8:
                old, new = int.from_bytes(want8, "little"), int.from_bytes(got, "little")
                _hits.append(
                    f"canary block of {size} bytes at {p:#x}, taken after '{label}', checked {when}: word at offset {off} "
                    f"is {new:#018x} instead of {old:#018x} (difference {new - old:+d}); first 32 bytes {raw[:32].hex()}")
        tail = raw[size - size % 8:]
        if tail.count(FILL) != len(tail):
            _hits.append(f"canary block of {size} bytes at {p:#x}, taken after '{label}', checked {when}: tail bytes {tail.hex()}")


def release_older_than(keep: int, when: str) -> None:
    """Check and free all but the newest `keep` generations."""
    before = len(_hits)
    while len(_generations) > keep:
        label, blocks = _generations.pop(0)
        _check(label, blocks, when)
        for p, _ in blocks:
            _libc.free(p)
    if len(_hits) > before:
        _write(_hits[before:])


def note(text: str) -> None:
    """A finding made elsewhere (a regenerated index structure) goes into the same report."""
    _hits.append(text)
    _write([text])


def _write(lines) -> None:
    path = os.environ.get("ET_CANARY_REPORT")
    if path:
        with open(path, "a") as f:
            for ln in lines:
                f.write(ln + "\n")


def report() -> list:
    return list(_hits)
