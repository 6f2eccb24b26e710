"""Write tests/golden/e8p_basis.npy from the reference's own basis().

Run once, in the container that holds /root/reference, as
    python tests/golden/make_basis_golden.py
Only the row ORDER of the 256x8 basis needs this: the value set, class counts,
parity rule and uniqueness of the 65 536 decoded vectors are fixed by closed
forms, but the order of rows comes solely from the reference source text
(python/orinfer_build/quantization/e8p.py:15-25).  The fixture is data: the
2 KiB int8 table itself, nothing of the reference's code.
"""
import sys
from pathlib import Path

import numpy as np

sys.path.insert(0, "/root/reference/python")
from orinfer_build.quantization.e8p import basis  # noqa: E402

table = basis()
assert table.shape == (256, 8) and table.dtype == np.int8
out = Path(__file__).with_name("e8p_basis.npy")
np.save(out, table)
print("wrote", out, table.shape, table.dtype)
