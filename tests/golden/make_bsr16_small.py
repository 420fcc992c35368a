"""Writes bsr16_small.json: expected BSR structure of two small matrices, stated by hand.

Matrix A (32 x 48, 2 x 3 tiles): tile (0,1) and tile (1,0), (1,2) non-zero.
Matrix B (48 x 32, 3 x 2 tiles): block-row 1 empty; tile (0,0), (0,1), (2,1) non-zero,
where tile (0,1) holds a single non-zero element (a tile is kept iff ANY element is non-zero).
"""
import json
from pathlib import Path

cases = {
    "A": {"shape": [32, 48], "nonzero_tiles": [[0, 1], [1, 0], [1, 2]],
          "row_ptr": [0, 1, 3], "column": [1, 0, 2]},
    "B": {"shape": [48, 32], "nonzero_tiles": [[0, 0], [0, 1], [2, 1]], "single_element_tiles": [[0, 1]],
          "row_ptr": [0, 2, 2, 3], "column": [0, 1, 1]},
}
Path(__file__).with_name("bsr16_small.json").write_text(json.dumps(cases, indent=1) + "\n")
