"""Weight exporter: a PyTorch-style state dict -> ``weights.txt`` + one ``.npz`` per layer, the
on-disk format the loader (``Weights`` / ``et_model_load``) reads.

File format and naming follow the reference exporter (example/npy2pt.py:112-174):
  * entry name = state-dict key minus its ``weight`` / ``bias`` suffix (so
    ``...self_attn.in_proj_``, ``...out_proj.``, ``...norm1.``, ``decoder.``), file ``<name>.npz``;
  * 2-D weight: ``row_ptr`` int32[out/16+1], ``column`` int32[ntile], ``data`` float32[ntile, 256],
    ``B`` float32[out] — 16x16 BSR of the [out, in] matrix, block-rows in order, column tiles
    ascending, a tile kept iff any element is non-zero (example/npy2pt.py:75-109);
  * 1-D weight (LayerNorm): ``W`` float32[H], ``B`` float32[H];
  * ``weights.txt``: one ``<name>.npz`` per line.
The BSR conversion is the library's host routine ``et_fmt_dense_to_bsr16`` (no GPU needed).

    python scpaper-2021_amd/export.py model.pt out_dir     # needs torch to read the checkpoint
"""
from __future__ import annotations

import ctypes as C
import sys
from pathlib import Path

import numpy as np

try:  # package import (scpaper_2021_amd.export) or plain script
    from . import check, lib
except ImportError:  # pragma: no cover - script use
    sys.path.insert(0, str(Path(__file__).resolve().parent.parent))
    import __graft_entry__ as _entry

    _pkg = _entry.load_package()
    check, lib = _pkg.check, _pkg.lib

SKIP_KEYS = ("encoder.weight", "pos_encoder.pe")  # embedding table and positional buffer (npy2pt.py:143-145)


def dense_to_bsr16(W: np.ndarray):
    """16x16 BSR arrays of a dense [out, in] matrix (both multiples of 16)."""
    W = np.ascontiguousarray(W, np.float32)
    nrow, ncol = W.shape
    if nrow % 16 or ncol % 16:
        raise ValueError(f"weight shape {W.shape} is not a multiple of 16")
    total = (nrow // 16) * (ncol // 16)
    row_ptr = np.zeros(nrow // 16 + 1, np.int32)
    column = np.zeros(max(total, 1), np.int32)
    data = np.zeros((max(total, 1), 256), np.float32)
    ntile = C.c_int()
    check(lib().et_fmt_dense_to_bsr16(W.ctypes.data, nrow, ncol, row_ptr.ctypes.data, column.ctypes.data,
                                      data.ctypes.data, C.byref(ntile)))
    n = ntile.value
    return row_ptr, column[:n].copy(), data[:n].copy()


def save_layer(path: str | Path, W: np.ndarray, B: np.ndarray) -> None:
    """One ``<name>.npz`` (np.savez appends the suffix)."""
    if W.ndim == 2:
        row_ptr, column, data = dense_to_bsr16(W)
        np.savez(str(path), row_ptr=row_ptr, column=column, data=data, B=np.asarray(B, np.float32))
    else:
        np.savez(str(path), W=np.asarray(W, np.float32), B=np.asarray(B, np.float32))


def export_state_dict(state_dict, folder: str | Path) -> list[str]:
    """Writes every (weight, bias) pair of ``state_dict`` and ``weights.txt``; returns the names."""
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    pairs: dict[str, list] = {}
    for key, value in state_dict.items():
        if key in SKIP_KEYS:
            continue
        arr = np.asarray(value.detach().cpu().numpy() if hasattr(value, "detach") else value)
        if key.endswith("weight"):
            pairs.setdefault(key[:-6], [None, None])[0] = arr
        elif key.endswith("bias"):
            pairs.setdefault(key[:-4], [None, None])[1] = arr
        else:
            raise ValueError(f"state-dict key {key!r} is neither a weight nor a bias")
    names = []
    for name, (W, B) in pairs.items():
        if W is None:
            raise ValueError(f"{name!r} has a bias but no weight")
        if B is None:
            B = np.zeros(W.shape[0], np.float32)
        save_layer(folder / name, W, B)
        names.append(f"{name}.npz")
    (folder / "weights.txt").write_text("".join(n + "\n" for n in names))
    return names


def main(argv=None) -> int:
    argv = sys.argv[1:] if argv is None else argv
    if len(argv) != 2:
        print(__doc__)
        return 2
    import torch

    sd = torch.load(argv[0], map_location="cpu", weights_only=True)
    names = export_state_dict(sd, argv[1])
    print(f"wrote {len(names)} archives and weights.txt to {argv[1]}")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
