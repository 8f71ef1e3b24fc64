"""Loads the golden vectors extracted from the reference's own tests."""

import json
import pathlib

import numpy as np

GOLDEN = pathlib.Path(__file__).resolve().parent / "golden"


def load(name):
    payload = json.loads((GOLDEN / name).read_text())
    return [np.array(item["value"]) for item in payload["arrays"]]
