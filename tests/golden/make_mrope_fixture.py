"""Writes tests/golden/mrope_positions.json from the two HF-generated data
fixtures the reference keeps under tests/resources (arrays only: input token
types, image grids and the expected 3-axis rope positions).  Run in the build
container, where /root/reference is mounted:

    python tests/golden/make_mrope_fixture.py
"""
import json
import os

import numpy as np

SRC = "/root/reference/tests/resources"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "mrope_positions.json")

IMAGE_TOKEN_TYPE = 1


def main() -> None:
    cases = []
    for name in ("qwen3_5_0.8B_ref.npz", "qwen3_5_0.8B_ref_2img.npz"):
        data = np.load(os.path.join(SRC, name))  # allow_pickle stays False
        ids = data["input_ids"].astype(np.int64)
        if "mm_token_type_ids" in data.files:
            types = data["mm_token_type_ids"].astype(np.int64)
        else:
            # the 2-image file stores no type ids: image placeholder tokens are the id
            # that the 1-image file marks with type 1
            one = np.load(os.path.join(SRC, "qwen3_5_0.8B_ref.npz"))
            image_id = int(one["input_ids"][one["mm_token_type_ids"] == IMAGE_TOKEN_TYPE][0])
            types = (ids == image_id).astype(np.int64)
        cases.append({
            "source": name,
            "mm_token_type_ids": types.tolist(),
            "image_grid_thw": data["image_grid_thw"].astype(np.int64).tolist(),
            "spatial_merge_size": 2,
            "rope_positions": data["rope_positions"].astype(np.int64).tolist(),
        })
    with open(OUT, "w") as f:
        json.dump(cases, f, indent=1)
    print(OUT)


if __name__ == "__main__":
    main()
