"""Writes tests/golden/codecs/deepseek_v4_fp4_expert.npz: the FP4 routed expert of the reference's
tests/fixtures/codecs/deepseek_v4_release.npz (the V4-Flash and V4.1-Flash releases' own conversion over a tiny
checkpoint, which tests/test_codecs.py:219-237 of the reference holds its decode to), copied as data: the stored nibbles
`[out, in / 2]`, their E8M0 scales `[out, in / 32]` and the release's dense reading `[out, in]` fp32.

    python tests/golden/make_deepseek_v4_fp4_expert.py /root/reference
"""

import sys
from pathlib import Path

import numpy as np

STORED = "stored/model.layers.0.mlp.experts.0.w1"


def main(reference: str) -> None:
    with np.load(Path(reference) / "tests/fixtures/codecs/deepseek_v4_release.npz", allow_pickle=False) as held:
        kept = {}
        for release in ("v4", "v4_1"):
            kept[f"{release}/weight"] = held[f"{release}/{STORED}.weight"]
            kept[f"{release}/scale"] = held[f"{release}/{STORED}.weight_scale_inv"]
            kept[f"{release}/dense"] = held[f"{release}/expert/dense"]
    np.savez_compressed(Path(__file__).parent / "codecs" / "deepseek_v4_fp4_expert.npz", **kept)


if __name__ == "__main__":
    main(sys.argv[1])
