"""Writes the small fixtures under tests/golden/ (run from the repo root: python tests/golden/make_fixtures.py).

Nothing here imports or runs the reference.  Two kinds of data:
  * compaction_cases.json — literal known answers.  Case "reference_docstring" is the worked example
    printed in the reference's docstring (flash_dropout/functional/utils.py:36-56), typed in by hand;
    the other cases were worked out by hand from the definitions (utils.py:57-67) and cover what that
    code special-cases: a fully dropped trailing row (:64-67), a fully dropped middle row, everything
    kept, everything dropped, a single row and a single column.
  * cfg1_mask.json — the 16x16 block mask of the CPU configuration (X, W, dY drawn first, then
    rand(16,16) < 0.5, all from torch.manual_seed(0) on the CPU generator), stored so that tests do
    not depend on the draw order.
"""
import json
from pathlib import Path

import torch

HERE = Path(__file__).resolve().parent

CASES = {
    "reference_docstring": {
        "block_k": 16,
        "mask": [[0, 1, 1, 0, 1], [1, 0, 0, 1, 0], [0, 1, 0, 1, 1]],
        "offsets": [0, 48, 16, 32, 64, 0, 32],
        "table": [0, 48, 16, 16, 32, 0, 32],
        "row_indices": [0, 2, 5],
        "row_widths": [2, 3, 2],
        "row_ptr": [0, 2, 5, 7],
        "col_idx": [0, 3, 1, 2, 4, 0, 2],
        "col_ptr": [0, 2, 3, 5, 6, 7],
        "row_idx": [0, 2, 1, 1, 2, 0, 1],
    },
    "trailing_row_dropped": {
        "block_k": 64,
        "mask": [[0, 0, 1], [1, 0, 0], [1, 1, 1]],
        "offsets": [0, 64, 64, 128],
        "table": [0, 64, 64, 64],
        "row_indices": [0, 2, 4],
        "row_widths": [2, 2, 0],
        "row_ptr": [0, 2, 4, 4],
        "col_idx": [0, 1, 1, 2],
        "col_ptr": [0, 1, 3, 4],
        "row_idx": [0, 0, 1, 1],
    },
    "middle_row_dropped": {
        "block_k": 8,
        "mask": [[1, 0], [1, 1], [0, 0]],
        "offsets": [8, 0, 8],
        "table": [8, 0, 8],
        "row_indices": [0, 1, 1],
        "row_widths": [1, 0, 2],
        "row_ptr": [0, 1, 1, 3],
        "col_idx": [1, 0, 1],
        "col_ptr": [0, 1, 3],
        "row_idx": [2, 0, 2],
    },
    "all_kept": {
        "block_k": 32,
        "mask": [[0, 0, 0], [0, 0, 0]],
        "offsets": [0, 32, 64, 0, 32, 64],
        "table": [0, 32, 32, 0, 32, 32],
        "row_indices": [0, 3],
        "row_widths": [3, 3],
        "row_ptr": [0, 3, 6],
        "col_idx": [0, 1, 2, 0, 1, 2],
        "col_ptr": [0, 2, 4, 6],
        "row_idx": [0, 1, 0, 1, 0, 1],
    },
    "all_dropped": {
        "block_k": 32,
        "mask": [[1, 1], [1, 1]],
        "offsets": [],
        "table": [],
        "row_indices": [0, 0],
        "row_widths": [0, 0],
        "row_ptr": [0, 0, 0],
        "col_idx": [],
        "col_ptr": [0, 0, 0],
        "row_idx": [],
    },
    "single_row": {
        "block_k": 4,
        "mask": [[1, 0, 0, 1, 0]],
        "offsets": [4, 8, 16],
        "table": [4, 4, 8],
        "row_indices": [0],
        "row_widths": [3],
        "row_ptr": [0, 3],
        "col_idx": [1, 2, 4],
        "col_ptr": [0, 0, 1, 2, 2, 3],
        "row_idx": [0, 0, 0],
    },
    "single_column": {
        "block_k": 4,
        "mask": [[0], [1], [0]],
        "offsets": [0, 0],
        "table": [0, 0],
        "row_indices": [0, 1, 1],
        "row_widths": [1, 0, 1],
        "row_ptr": [0, 1, 1, 2],
        "col_idx": [0, 0],
        "col_ptr": [0, 2],
        "row_idx": [0, 2],
    },
}


def cfg1_mask():
    torch.manual_seed(0)
    torch.randn(1024, 1024)  # X
    torch.randn(1024, 1024)  # W (scaled by 1/32 by the user of the fixture)
    torch.randn(1024, 1024)  # dY
    return torch.rand(16, 16) < 0.5


if __name__ == "__main__":
    (HERE / "compaction_cases.json").write_text(json.dumps(CASES, indent=1) + "\n")
    m = cfg1_mask()
    (HERE / "cfg1_mask.json").write_text(json.dumps({
        "block_size": 64, "p": 0.5, "seed": 0, "shape": [16, 16],
        "order": "torch.manual_seed(0); randn X[1024,1024]; randn W[1024,1024]; randn dY[1024,1024]; rand(16,16) < 0.5",
        "rows": ["".join("1" if v else "0" for v in row) for row in m.tolist()],
    }, indent=1) + "\n")
    print("kept blocks:", int((~m).sum()))
