"""Writes tests/golden/packing.json: hand-derived known answers for the two
packed formats.  The expected bytes below were worked out by hand from the
format definition (element i -> byte i//8, bit 7-(i%8); element 2j -> high
nibble of byte j), not by running any implementation."""
import json
from pathlib import Path

FIXTURES = {
    "pack_bits": [
        # bits, expected bytes
        {"bits": [1, 0, 1, 1, 0, 0, 0, 1, 1, 1], "bytes": [0xB1, 0xC0]},
        {"bits": [1], "bytes": [0x80]},
        {"bits": [0, 0, 0, 0, 0, 0, 0, 1], "bytes": [0x01]},
        {"bits": [0, 1, 0, 1, 0, 1, 0, 1, 1, 0, 1, 0, 1, 0, 1, 0, 1, 1, 1], "bytes": [0x55, 0xAA, 0xE0]},
        {"bits": [1] * 16, "bytes": [0xFF, 0xFF]},
        {"bits": [0] * 9, "bytes": [0x00, 0x00]},
    ],
    "pack_nibbles": [
        {"values": [1, 2, 3], "bytes": [0x12, 0x30]},
        {"values": [15, 0, 0, 15], "bytes": [0xF0, 0x0F]},
        {"values": [8], "bytes": [0x80]},
        {"values": [0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15],
         "bytes": [0x01, 0x23, 0x45, 0x67, 0x89, 0xAB, 0xCD, 0xEF]},
    ],
    # 1x1x4x4 input, 3x3 s2 p1 max pool: windows and hand-derived results.
    # rows: [1 2 3 4],[5 6 7 8],[9 9 1 0],[2 9 3 3]
    # out(0,0): window rows -1..1, cols -1..1 -> valid {1,2,5,6} max 6 at (h1,w1) -> ch=2,cw=2 -> 8
    # out(0,1): rows -1..1, cols 1..3 -> {2,3,4,6,7,8} max 8 at (h1,w3) -> ch=2,cw=2 -> 8
    # out(1,0): rows 1..3, cols -1..1 -> {5,6,9,9,2,9}: first 9 at (h2,w0) -> ch=1,cw=1 -> 4
    # out(1,1): rows 1..3, cols 1..3 -> {6,7,8,9,1,0,9,3,3}: first 9 at (h2,w1) -> ch=1,cw=0 -> 3
    "maxpool_3x3_s2_p1": {
        "x": [[1, 2, 3, 4], [5, 6, 7, 8], [9, 9, 1, 0], [2, 9, 3, 3]],
        "y": [[6, 8], [9, 9]],
        "idx": [[8, 8], [4, 3]],
        "packed": [0x88, 0x43],
        # dy = [[1,2],[3,4]] scattered: 6@(1,1)<-1 ; 8@(1,3)<-2 ; 9@(2,0)<-3 ; 9@(2,1)<-4
        "dy": [[1, 2], [3, 4]],
        "dx": [[0, 0, 0, 0], [0, 1, 0, 2], [3, 4, 0, 0], [0, 0, 0, 0]],
    },
}

if __name__ == "__main__":
    out = Path(__file__).resolve().parent / "packing.json"
    out.write_text(json.dumps(FIXTURES, indent=1))
    print("wrote", out)
