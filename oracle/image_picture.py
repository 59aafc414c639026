"""CPU restatement of the reference's array-backed image front-end (OpenCVPicture),
TEST INFRASTRUCTURE ONLY: nothing in the product imports this file.

  codify  OpenCVPicture.cpp:368-402 with the offsets of the constructor, :9-15, and
          scaleUCharColor, :4-7
Pins (tests/test_image_picture.py): hand-computed images (cell arithmetic with the
constructor's offsets, the > 2 threshold per channel, clipping at the field, column-major
insertion order, colour scaling for backgrounds 0, 128 and 200).
"""
import numpy as np


def codify(pixels, backgroundColor, spatialSize, xOffset=None, yOffset=None):
    """pixels [rows x cols x channels], values 0..255.
    -> (keys in insertion order, rows, background row, features [rows x channels])."""
    px = np.asarray(pixels, np.float32)
    if px.ndim == 2:
        px = px[:, :, None]
    rows, cols, ch = px.shape
    # the constructor is called (xSize, ySize) and makes xSize the row count
    xOffset = -(rows // 2) if xOffset is None else xOffset
    yOffset = -(cols // 2) if yOffset is None else yOffset
    S = spatialSize
    bg = np.float32(backgroundColor)
    div = np.float32(max(255 - backgroundColor, backgroundColor))
    x0, x1 = max(0, -xOffset - S // 2), min(cols, S - xOffset - S // 2)
    y0, y1 = max(0, -yOffset - S // 2), min(rows, S - yOffset - S // 2)
    keys, feats = [], [np.zeros(ch, np.float32)]
    for x in range(x0, x1):
        for y in range(y0, y1):
            v = px[y, x]
            if np.any(np.abs(v - bg) > 2):
                keys.append((x + xOffset + S // 2) * S + (y + yOffset + S // 2))
                feats.append((v - bg) / div)
    keys = np.array(keys, np.int64)
    return keys, np.arange(1, len(keys) + 1, dtype=np.int32), 0, np.stack(feats).astype(np.float32)
