"""Writes tests/golden/model_logits.npz: the logits of the full-size ResNet-50 and MobileNetV2 .one models (batch 1,
seeded input) as the reference's own host operator classes and x86 kernels compute them (oracle/_ref/ref_run_one,
built by `make -C oracle ref` where the reference sources are mounted).  The GPU tests compare the device-resident
runtime with these vectors, so they need neither the reference nor its build.

    python tests/golden/make_model_logits.py
"""
import hashlib
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from onenew_amd import datagen, stacks      # noqa: E402
from oracle import one_model                # noqa: E402

OUT = os.path.join(HERE, "model_logits.npz")


def model_and_input(model):
    """the .one file and the input the fixture was made with"""
    make = stacks.resnet50_model if model == "resnet50" else stacks.mobilenet_v2_model
    data, shape, _ = make(1)
    x = datagen.normal(datagen.seed_for("model_logits", model, "x"), shape, 0.0, 1.0)
    return data, x


def main():
    if not one_model.have_ref_runner():
        raise SystemExit("oracle/_ref/ref_run_one is missing: run `make -C oracle ref` where /root/reference is mounted")
    out = {}
    for model in ("resnet50", "mobilenetv2"):
        data, x = model_and_input(model)
        (_, logits), = one_model.run_reference(data, [x])
        out[model + "_logits"] = logits.astype(np.float32)
        out[model + "_sha256"] = np.frombuffer(hashlib.sha256(data).digest(), dtype=np.uint8)
        print(model, logits.shape, "top-5", np.argsort(logits[0])[-5:][::-1], "max |logit|", float(np.abs(logits).max()))
    np.savez_compressed(OUT, **out)
    print("wrote", OUT)


if __name__ == "__main__":
    main()
