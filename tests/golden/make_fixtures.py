"""Regenerates the data fixtures under tests/golden/ from the reference checkout (run in the build
container, where /root/reference exists; the GPU box only ever sees the committed outputs).

  squeezenet_whole/graph.dr, N.var   the stored SqueezeNet v1.1 model the reference ships as its
                                     example (examples/squeezenet-v1.1/squeezenet_whole/): topology
                                     text + raw little-endian fp32 weights.  Data, copied byte for byte.
                                     The generated .cl kernel texts in that folder are NOT copied.
  tiger_224_rgb_u8.npy, puzzle_224_rgb_u8.npy
                                     the two 224x224 RGB example images, decoded with PIL to uint8
                                     [H][W][3]; expected classes 292 and 611
                                     (examples/squeezenet-v1.1/squeezenet_deployed.c:199-207).
"""
import os
import shutil
import sys

import numpy as np
from PIL import Image

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))
src = os.path.join(REF, "examples", "squeezenet-v1.1")
dst = os.path.join(HERE, "squeezenet_whole")
os.makedirs(dst, exist_ok=True)
for f in sorted(os.listdir(os.path.join(src, "squeezenet_whole"))):
    if f == "graph.dr" or f.endswith(".var"):
        shutil.copyfile(os.path.join(src, "squeezenet_whole", f), os.path.join(dst, f))
for name in ("tiger", "puzzle"):
    img = np.asarray(Image.open(os.path.join(src, name + ".png")).convert("RGB"), dtype=np.uint8)
    assert img.shape == (224, 224, 3)
    np.save(os.path.join(HERE, "%s_224_rgb_u8.npy" % name), img)
print("fixtures written to", HERE)
