"""Write golden block -> value fixtures with the reference's own numpy decoders.

Run ONLY in the build container, where the reference checkout is mounted:

    python tests/golden/make_reference_fixtures.py /root/reference

It imports the reference's GGUF reader from that checkout, feeds it seeded random blocks of the types
that no reference-held vector and no compiled reference kernel pins (Q8_0, Q4_K, Q5_K, Q6_K, IQ4_XS, IQ2_XS, IQ3_XXS, Q3_K, and
IQ2_XXS, whose compiled CPU kernel takes the sign-expanded grid from its caller) through a one-tensor GGUF file
in a temporary directory, and stores {blocks, values} as hex in JSON files next to this script, plus
SHA-256 digests of the two codebook arrays the reference builds (sign-expanded IQ2_XXS grid, IQ1 grid).  The fixtures are data; the reference itself never leaves the container.
"""
from __future__ import annotations

import json
import struct
import sys
import tempfile
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
GGML_TYPE = {"q8_0": 8, "q4_k": 12, "q5_k": 13, "iq2_xxs": 16, "q6_k": 14, "iq4_xs": 23, "iq2_xs": 17, "iq3_xxs": 18, "q3_k": 11}
GEOM = {"q8_0": (32, 34), "q4_k": (256, 144), "q5_k": (256, 176), "iq2_xxs": (256, 66), "q6_k": (256, 210), "iq4_xs": (256, 136), "iq2_xs": (256, 74), "iq3_xxs": (256, 98), "q3_k": (256, 110)}
F16_FIELDS = {"q8_0": [0], "q4_k": [0, 2], "q5_k": [0, 2], "iq2_xxs": [0], "q6_k": [208], "iq4_xs": [0], "iq2_xs": [0], "iq3_xxs": [0], "q3_k": [108]}
ROWS, BLOCKS_PER_ROW = 3, 2


def _pack_string(s: str) -> bytes:
    b = s.encode("utf-8")
    return struct.pack("<Q", len(b)) + b


def write_one_tensor_gguf(path: Path, name: str, dims, type_id: int, payload: bytes) -> None:
    buf = bytearray()
    buf += b"GGUF"
    buf += struct.pack("<I", 3)
    buf += struct.pack("<Q", 1)
    buf += struct.pack("<Q", 0)
    buf += _pack_string(name)
    buf += struct.pack("<I", len(dims))
    for d in dims:
        buf += struct.pack("<Q", int(d))
    buf += struct.pack("<I", int(type_id))
    buf += struct.pack("<Q", 0)
    while len(buf) % 32:
        buf += b"\0"
    buf += payload
    path.write_bytes(bytes(buf))


def random_blocks(rng: np.random.Generator, type_name: str) -> np.ndarray:
    elems, nbytes = GEOM[type_name]
    blocks = rng.integers(0, 256, size=(ROWS, BLOCKS_PER_ROW, nbytes), dtype=np.uint8)
    for off in F16_FIELDS[type_name]:
        # finite, sign-mixed fp16 scale fields
        vals = (rng.uniform(0.001, 0.05, size=(ROWS, BLOCKS_PER_ROW)) * rng.choice([-1.0, 1.0], size=(ROWS, BLOCKS_PER_ROW)))
        blocks[..., off:off + 2] = vals.astype("<f2").view(np.uint8).reshape(ROWS, BLOCKS_PER_ROW, 2)
    return blocks


def main() -> None:
    ref_root = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    sys.path.insert(0, str(ref_root))
    from src.loader.gguf.tensor_reader import GGUFTensorDataReader  # the reference's decoders

    rng = np.random.default_rng(20240607)
    with tempfile.TemporaryDirectory() as tmp:
        for type_name in ("q8_0", "q4_k", "q5_k", "iq2_xxs", "q6_k", "iq4_xs", "iq2_xs", "iq3_xxs", "q3_k"):      # new types go last: the stream of random blocks of the earlier ones stays the same
            elems, nbytes = GEOM[type_name]
            blocks = random_blocks(rng, type_name)
            path = Path(tmp) / f"{type_name}.gguf"
            write_one_tensor_gguf(path, "w", (BLOCKS_PER_ROW * elems, ROWS), GGML_TYPE[type_name], blocks.tobytes())
            with GGUFTensorDataReader(str(path)) as reader:
                values = reader.read_tensor("w").numpy().astype("<f4")
            assert values.shape == (ROWS, BLOCKS_PER_ROW * elems)
            out = {
                "type": type_name,
                "rows": ROWS,
                "blocks_per_row": BLOCKS_PER_ROW,
                "block_bytes": nbytes,
                "block_elems": elems,
                "blocks_u8": blocks.tobytes().hex(),
                "values_f32": values.tobytes().hex(),
                "made_by": "reference GGUFTensorDataReader.read_tensor (src/loader/gguf/tensor_reader.py)",
            }
            (HERE / f"{type_name}_reference_decode.json").write_text(json.dumps(out), encoding="utf-8")
            print(type_name, "ok", values.shape)

    import hashlib
    from src.loader.gguf.iq1_grid import iq1_grid_i8
    from src.loader.gguf.tensor_reader import _iq2xxs_signed_grid

    signed = np.ascontiguousarray(_iq2xxs_signed_grid())
    iq1 = np.ascontiguousarray(iq1_grid_i8())
    digests = {
        "iq2xxs_signed_grid": {"shape": list(signed.shape), "dtype": str(signed.dtype),
                               "sha256": hashlib.sha256(signed.tobytes()).hexdigest()},
        "iq1_grid_i8": {"shape": list(iq1.shape), "dtype": str(iq1.dtype),
                        "sha256": hashlib.sha256(iq1.tobytes()).hexdigest()},
    }
    (HERE / "codebook_digests.json").write_text(json.dumps(digests, indent=1), encoding="utf-8")
    print("codebook digests ok")


if __name__ == "__main__":
    main()
