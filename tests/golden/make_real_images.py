"""Decodes eight images of the reference's own test data (data/images/AMD-tinyDataSet/*.JPEG, 299 x 299 RGB: what
tests/cpp_api/CMakeLists.txt:83-253 feeds its unit tests) with Pillow and writes their raw pixels to
tests/golden/amd_tiny_8.npz. The file holds DATA of the reference (decoded pixels), labelled with its source; decoders
are outside the hot path, so which JPEG decoder produced the bytes does not matter to the tests that use them: they compare
this library's kernels with the oracle on the same pixels. Run in the build container (the reference tree is not on the GPU box):
  python tests/golden/make_real_images.py
"""
import glob
import os

import numpy as np
from PIL import Image

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = "/root/reference/data/images/AMD-tinyDataSet"


def main():
    files = sorted(glob.glob(os.path.join(SRC, "*.JPEG")))
    picked = files[::len(files) // 8][:8]  # spread over the data set
    images = np.stack([np.asarray(Image.open(f).convert("RGB"), dtype=np.uint8) for f in picked])
    assert images.shape == (8, 299, 299, 3), images.shape
    np.savez_compressed(os.path.join(HERE, "amd_tiny_8.npz"), images=images, files=np.array([os.path.basename(f) for f in picked]),
                        source=np.array("decoded with Pillow from /root/reference/data/images/AMD-tinyDataSet (rocAL test data)"))
    print(images.shape, os.path.getsize(os.path.join(HERE, "amd_tiny_8.npz")))


if __name__ == "__main__":
    main()
