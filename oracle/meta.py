"""Bounding-box metadata laws of the hot-path nodes, restated for checking (test infrastructure only).

Pure Python over numpy float32 scalars: every operation is rounded to fp32 in the reference's order.
Follows rocAL/include/meta_data/meta_node.h:42-60 (intersection test) and rocAL/source/meta_data/
meta_node_{crop,crop_mirror_normalize,crop_resize,resize,resize_crop_mirror,resize_mirror_normalize,flip,rotate}.cpp.
A box is (l, t, r, b); a sample is a list of boxes plus a list of labels.
"""
import math

import numpy as np

F = np.float32
IOU_THRESHOLD = F(0.25)  # meta_node.h:39


def _box(b):
    return tuple(F(v) for v in b)


def overlap(box1, box2, is_iou=False):
    """meta_node.h:42-60: intersection over the first box's area (over the union when is_iou)."""
    xa, ya = max(box1[0], box2[0]), max(box1[1], box2[1])
    xb, yb = min(box1[2], box2[2]), min(box1[3], box2[3])
    inter = F(max(F(0), F(xb - xa)) * max(F(0), F(yb - ya)))
    a1 = F(F(box1[3] - box1[1]) * F(box1[2] - box1[0]))
    a2 = F(F(box2[3] - box2[1]) * F(box2[2] - box2[0]))
    with np.errstate(divide="ignore", invalid="ignore"):
        if is_iou:
            return float(F(inter / F(F(a1 + a2) - inter)))
        return float(F(inter / a1))


def _crop_boxes(boxes, labels, crop_box, fallback, finish):
    out_b, out_l = [], []
    crop_box = _box(crop_box)
    for b, lab in zip(boxes, labels):
        b = _box(b)
        if overlap(b, crop_box) >= float(IOU_THRESHOLD):
            xa, ya = max(crop_box[0], b[0]), max(crop_box[1], b[1])
            xb, yb = min(crop_box[2], b[2]), min(crop_box[3], b[3])
            nb = [F(xa - crop_box[0]), F(ya - crop_box[1]), F(xb - crop_box[0]), F(yb - crop_box[1])]
            finish(nb)
            out_b.append(tuple(nb))
            out_l.append(lab)
    if not out_b:
        out_b.append(_box(fallback))
        out_l.append(0)
    return out_b, out_l


def crop(boxes, labels, x1, y1, w, h):
    """meta_node_crop.cpp:44-78"""
    return _crop_boxes(boxes, labels, (x1, y1, x1 + w, y1 + h), (0, 0, w, h), lambda b: None)


def crop_mirror_normalize(boxes, labels, x1, y1, w, h, mirror):
    """meta_node_crop_mirror_normalize.cpp:49-86"""
    def finish(b):
        if mirror == 1:
            l = b[0]
            b[0] = F(F(w) - b[2])
            b[2] = F(F(w) - l)
    return _crop_boxes(boxes, labels, (x1, y1, x1 + w, y1 + h), (0, 0, w, h), finish)


def _scale(b, wr, hr):
    b[0], b[1], b[2], b[3] = F(b[0] * wr), F(b[1] * hr), F(b[2] * wr), F(b[3] * hr)


def crop_resize(boxes, labels, x1, y1, x2, y2, resize_w, resize_h):
    """meta_node_crop_resize.cpp:45-85"""
    cw, ch = x2 - x1, y2 - y1
    wr, hr = F(F(resize_w) / F(cw)), F(F(resize_h) / F(ch))
    return _crop_boxes(boxes, labels, (x1, y1, x1 + cw, y1 + ch), (0, 0, resize_w, resize_h), lambda b: _scale(b, wr, hr))


def resize_crop_mirror(boxes, labels, x1, y1, x2, y2, resize_w, resize_h, mirror):
    """meta_node_resize_crop_mirror.cpp:51-100"""
    cw, ch = x2 - x1, y2 - y1
    wr, hr = F(F(resize_w) / F(cw)), F(F(resize_h) / F(ch))

    def finish(b):
        if mirror == 1:
            l = b[0]
            b[0] = F(F(cw) - b[2])
            b[2] = F(F(cw) - l)
        _scale(b, wr, hr)
    return _crop_boxes(boxes, labels, (x1, y1, x2, y2), (0, 0, resize_w, resize_h), finish)


def resize(boxes, labels, in_w, in_h, out_w, out_h):
    """meta_node_resize.cpp:31-54 (an empty sample gets a zero box and no label)"""
    wr, hr = F(F(out_w) / F(in_w)), F(F(out_h) / F(in_h))
    out = []
    for b in boxes:
        b = list(_box(b))
        _scale(b, wr, hr)
        out.append(tuple(b))
    if not out:
        out.append(_box((0, 0, 0, 0)))
    return out, list(labels)


def resize_mirror_normalize(boxes, labels, in_w, in_h, out_w, out_h, mirror):
    """meta_node_resize_mirror_normalize.cpp:37-85"""
    wr, hr = F(F(out_w) / F(in_w)), F(F(out_h) / F(in_h))
    out = []
    for b in boxes:
        b = list(_box(b))
        _scale(b, wr, hr)
        if mirror == 1:
            l = b[0]
            b[0] = F(F(F(out_w) - b[2]) - F(1))
            b[2] = F(F(F(out_w) - l) - F(1))
        out.append(tuple(b))
    return out, list(labels)


def flip(boxes, labels, in_w, in_h, h_flip, v_flip):
    """meta_node_flip.cpp:38-59"""
    out = []
    for b in boxes:
        b = list(_box(b))
        if h_flip:
            l = b[0]
            b[0] = F(F(in_w) - b[2])
            b[2] = F(F(in_w) - l)
        if v_flip:
            t = b[1]
            b[1] = F(F(in_h) - b[3])
            b[3] = F(F(in_h) - t)
        out.append(tuple(b))
    return out, list(labels)


def rotate(boxes, labels, in_w, in_h, dst_w, dst_h, angle_deg):
    """meta_node_rotate.cpp:38-96 (cos/sin evaluated in double and rounded to fp32)"""
    dest = _box((0, 0, dst_w, dst_h))
    out_b, out_l = [], []
    for b, lab in zip(boxes, labels):
        b = _box(b)
        radian = F(float(F(angle_deg)) * 3.14159265 / 180)
        c, s = F(math.cos(float(radian))), F(math.sin(float(radian)))
        r0, r1, r2, r3 = c, s, F(F(-1) * s), c
        dcx, dcy = F(dst_w // 2), F(dst_h // 2)
        scx, scy = F(F(in_w) / F(2)), F(F(in_h) / F(2))
        bx, by = b[0], b[1]
        bw, bh = F(b[2] - b[0]), F(b[3] - b[1])

        def pt(px, py):
            x = F(F(F(r0 * F(px - scx)) + F(r1 * F(py - scy))) + dcx)
            y = F(F(F(r2 * F(px - scx)) + F(r3 * F(py - scy))) + dcy)
            return x, y
        xs, ys = zip(pt(bx, by), pt(F(bx + bw), by), pt(bx, F(by + bh)), pt(F(bx + bw), F(by + bh)))
        box = (min(F(0), min(xs)), min(F(0), min(ys)), max(xs), max(ys))
        if overlap(box, dest) >= float(IOU_THRESHOLD):
            out_b.append((max(dest[0], box[0]), max(dest[1], box[1]), min(dest[2], box[2]), min(dest[3], box[3])))
            out_l.append(lab)
    if not out_b:
        out_b.append(dest)
        out_l.append(0)
    return out_b, out_l
