"""Re-pack the reference's golden tensors (data only) into one .npz fixture.

Source: /root/reference/test_data.zip, the 13 fp32 tensors that the reference's
own fixture scripts load (fhog/test_bwdbwd.py:27-51, fhog/jax_refs/torch_impl.py:205-226).
They are read with ``torch.load(weights_only=True)`` (nothing from the file is
executed) and written as plain float32 arrays.  No reference code is imported or run.

Shapes: q, o, do, ddq, dq2, ddo (128, 64); k, v, ddk, ddv, dk2, dv2 (256, 64); L (128,).
Non-causal, scale = 1/sqrt(64).

Usage (only in the authoring container, where /root/reference exists):
    python tests/golden/extract_reference_fixture.py
"""
import io
import sys
import zipfile
from pathlib import Path

import numpy as np
import torch

ZIP = Path("/root/reference/test_data.zip")
OUT = Path(__file__).resolve().parent / "reference_test_data.npz"

INPUTS = ["q", "k", "v", "o", "L", "do", "ddq", "ddk", "ddv"]
OUTPUTS = ["dq2", "dk2", "dv2", "ddo"]


def main() -> int:
    arrays = {}
    with zipfile.ZipFile(ZIP) as z:
        for group, names in (("input_items", INPUTS), ("output_items", OUTPUTS)):
            for n in names:
                raw = z.read(f"test_data/{group}/{n}.pt")
                t = torch.load(io.BytesIO(raw), weights_only=True, map_location="cpu")
                assert t.dtype == torch.float32, (n, t.dtype)
                arrays[n] = t.numpy().copy()
    np.savez_compressed(OUT, **arrays)
    for n, a in arrays.items():
        print(f"{n:4s} {a.shape} {a.dtype}")
    print("wrote", OUT, OUT.stat().st_size, "bytes")
    return 0


if __name__ == "__main__":
    sys.exit(main())
