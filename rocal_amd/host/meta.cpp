#include "meta.h"

#include <algorithm>
#include <cmath>

double MetaNode::BBoxIntersectionOverUnion(const BoundingBoxCord &box1, const BoundingBoxCord &box2, bool is_iou) const {
    const float xA = std::max(box1.l, box2.l), yA = std::max(box1.t, box2.t);
    const float xB = std::min(box1.r, box2.r), yB = std::min(box1.b, box2.b);
    const float intersection_area = std::max(0.0f, xB - xA) * std::max(0.0f, yB - yA);
    const float box1_area = (box1.b - box1.t) * (box1.r - box1.l);
    const float box2_area = (box2.b - box2.t) * (box2.r - box2.l);
    if (is_iou) return intersection_area / float(box1_area + box2_area - intersection_area);
    return intersection_area / float(box1_area);
}

void BoundingBoxGraph::process(pMetaDataBatch input_meta_data, pMetaDataBatch output_meta_data) {
    size_t left = _meta_nodes.size();
    for (auto &meta_node : _meta_nodes) {
        meta_node->update_parameters(input_meta_data, output_meta_data);
        if (--left > 0) input_meta_data = output_meta_data->clone();
    }
}

namespace {

// The part shared by the crop-type nodes: keep the boxes that overlap the crop window enough, clip them to it
// and move them into its frame; `finish` applies what the node does after that (mirror, scale).
template <typename Finish>
void crop_boxes(const MetaNode &self, pMetaDataBatch in, pMetaDataBatch out, int i, const BoundingBoxCord &crop_box, const BoundingBoxCord &fallback,
                Finish finish) {
    const Labels labels_buf = in->get_labels_batch()[i];
    BoundingBoxCords coords_buf = in->get_bb_cords_batch()[i];
    BoundingBoxCords bb_coords;
    Labels bb_labels;
    for (size_t j = 0; j < labels_buf.size(); j++) {
        if (self.BBoxIntersectionOverUnion(coords_buf[j], crop_box) >= self._iou_threshold) {
            const float xA = std::max(crop_box.l, coords_buf[j].l), yA = std::max(crop_box.t, coords_buf[j].t);
            const float xB = std::min(crop_box.r, coords_buf[j].r), yB = std::min(crop_box.b, coords_buf[j].b);
            BoundingBoxCord box{xA - crop_box.l, yA - crop_box.t, xB - crop_box.l, yB - crop_box.t};
            finish(box);
            bb_coords.push_back(box);
            bb_labels.push_back(labels_buf[j]);
        }
    }
    if (bb_coords.empty()) {  // "all crops should at least have one box": the whole output with label 0
        bb_coords.push_back(fallback);
        bb_labels.push_back(0);
    }
    out->get_bb_cords_batch()[i] = bb_coords;
    out->get_labels_batch()[i] = bb_labels;
}

}  // namespace

void CropMetaNode::update_parameters(pMetaDataBatch in, pMetaDataBatch out) {
    auto p = _node->get_crop_param();
    for (int i = 0; i < (int)in->size(); i++) {
        const unsigned x1 = p->get_x1_arr_val()[i], y1 = p->get_y1_arr_val()[i], w = p->get_cropw_arr_val()[i], h = p->get_croph_arr_val()[i];
        const BoundingBoxCord crop_box{static_cast<float>(x1), static_cast<float>(y1), static_cast<float>(x1 + w), static_cast<float>(y1 + h)};
        crop_boxes(*this, in, out, i, crop_box, {0, 0, static_cast<float>(w), static_cast<float>(h)}, [](BoundingBoxCord &) {});
    }
}

void CropMirrorNormalizeMetaNode::update_parameters(pMetaDataBatch in, pMetaDataBatch out) {
    auto p = _node->get_crop_param();
    const std::vector<int> &mirror = _node->mirror_values();
    for (int i = 0; i < (int)in->size(); i++) {
        const unsigned x1 = p->get_x1_arr_val()[i], y1 = p->get_y1_arr_val()[i], w = p->get_cropw_arr_val()[i], h = p->get_croph_arr_val()[i];
        const BoundingBoxCord crop_box{static_cast<float>(x1), static_cast<float>(y1), static_cast<float>(x1 + w), static_cast<float>(y1 + h)};
        crop_boxes(*this, in, out, i, crop_box, {0, 0, static_cast<float>(w), static_cast<float>(h)}, [&](BoundingBoxCord &box) {
            if (mirror[i] == 1) {
                const float l = box.l;
                box.l = w - box.r;
                box.r = w - l;
            }
        });
    }
}

void CropResizeMetaNode::update_parameters(pMetaDataBatch in, pMetaDataBatch out) {
    const CropParam *p = _node->get_crop_param();
    const unsigned resize_w = _node->get_dst_width(), resize_h = _node->get_dst_height();
    for (int i = 0; i < (int)in->size(); i++) {
        const unsigned x1 = p->get_x1_arr_val()[i], y1 = p->get_y1_arr_val()[i];
        const unsigned crop_w = p->get_x2_arr_val()[i] - x1, crop_h = p->get_y2_arr_val()[i] - y1;
        const BoundingBoxCord crop_box{static_cast<float>(x1), static_cast<float>(y1), static_cast<float>(x1 + crop_w), static_cast<float>(y1 + crop_h)};
        const float wr = static_cast<float>(resize_w) / crop_w, hr = static_cast<float>(resize_h) / crop_h;
        crop_boxes(*this, in, out, i, crop_box, {0, 0, static_cast<float>(resize_w), static_cast<float>(resize_h)}, [&](BoundingBoxCord &box) {
            box.l *= wr;
            box.t *= hr;
            box.r *= wr;
            box.b *= hr;
        });
    }
}

void ResizeCropMirrorMetaNode::update_parameters(pMetaDataBatch in, pMetaDataBatch out) {
    auto p = _node->get_crop_param();
    const std::vector<int> &mirror = _node->mirror_values();
    const unsigned resize_w = _node->get_dst_width(), resize_h = _node->get_dst_height();
    for (int i = 0; i < (int)in->size(); i++) {
        const unsigned x1 = p->get_x1_arr_val()[i], y1 = p->get_y1_arr_val()[i], x2 = p->get_x2_arr_val()[i], y2 = p->get_y2_arr_val()[i];
        const unsigned crop_w = x2 - x1, crop_h = y2 - y1;
        const BoundingBoxCord crop_box{static_cast<float>(x1), static_cast<float>(y1), static_cast<float>(x2), static_cast<float>(y2)};
        const float wr = static_cast<float>(resize_w) / crop_w, hr = static_cast<float>(resize_h) / crop_h;
        crop_boxes(*this, in, out, i, crop_box, {0, 0, static_cast<float>(resize_w), static_cast<float>(resize_h)}, [&](BoundingBoxCord &box) {
            if (mirror[i] == 1) {
                const float l = box.l;
                box.l = crop_w - box.r;
                box.r = crop_w - l;
            }
            box.l *= wr;
            box.t *= hr;
            box.r *= wr;
            box.b *= hr;
        });
    }
}

void ResizeMetaNode::update_parameters(pMetaDataBatch in, pMetaDataBatch out) {
    const Roi2DCords *input_roi = _node->get_src_roi(), *output_roi = _node->get_dst_roi();
    for (int i = 0; i < (int)in->size(); i++) {
        const float wr = static_cast<float>(output_roi[i].xywh.w) / static_cast<float>(input_roi[i].xywh.w);
        const float hr = static_cast<float>(output_roi[i].xywh.h) / static_cast<float>(input_roi[i].xywh.h);
        BoundingBoxCords coords_buf = in->get_bb_cords_batch()[i];
        for (auto &c : coords_buf) {
            c.l *= wr;
            c.t *= hr;
            c.r *= wr;
            c.b *= hr;
        }
        out->get_labels_batch()[i] = in->get_labels_batch()[i];
        if (coords_buf.empty()) coords_buf.push_back({0, 0, 0, 0});  // (no label goes with it in the reference either)
        out->get_bb_cords_batch()[i] = coords_buf;
    }
}

void ResizeMirrorNormalizeMetaNode::update_parameters(pMetaDataBatch in, pMetaDataBatch out) {
    const Roi2DCords *input_roi = _node->get_src_roi(), *output_roi = _node->get_dst_roi();
    const std::vector<int> &mirror = _node->mirror_values();
    for (int i = 0; i < (int)in->size(); i++) {
        const float wr = static_cast<float>(output_roi[i].xywh.w) / static_cast<float>(input_roi[i].xywh.w);
        const float hr = static_cast<float>(output_roi[i].xywh.h) / static_cast<float>(input_roi[i].xywh.h);
        BoundingBoxCords coords_buf = in->get_bb_cords_batch()[i];
        for (auto &c : coords_buf) {
            c.l *= wr;
            c.t *= hr;
            c.r *= wr;
            c.b *= hr;
            if (mirror[i] == 1) {
                const float l = c.l;
                c.l = output_roi[i].xywh.w - c.r - 1;
                c.r = output_roi[i].xywh.w - l - 1;
            }
        }
        out->get_bb_cords_batch()[i] = coords_buf;
        out->get_labels_batch()[i] = in->get_labels_batch()[i];
    }
}

void FlipMetaNode::update_parameters(pMetaDataBatch in, pMetaDataBatch out) {
    const Roi2DCords *input_roi = _node->get_src_roi();
    const std::vector<int> &h_flip = _node->horizontal_values(), &v_flip = _node->vertical_values();
    for (int i = 0; i < (int)in->size(); i++) {
        BoundingBoxCords coords_buf = in->get_bb_cords_batch()[i];
        for (auto &c : coords_buf) {
            if (h_flip[i]) {
                const float l = c.l;
                c.l = input_roi[i].xywh.w - c.r;
                c.r = input_roi[i].xywh.w - l;
            }
            if (v_flip[i]) {
                const float t = c.t;
                c.t = input_roi[i].xywh.h - c.b;
                c.b = input_roi[i].xywh.h - t;
            }
        }
        out->get_bb_cords_batch()[i] = coords_buf;
        out->get_labels_batch()[i] = in->get_labels_batch()[i];
    }
}

void RotateMetaNode::update_parameters(pMetaDataBatch in, pMetaDataBatch out) {
    const Roi2DCords *input_roi = _node->get_src_roi();
    const unsigned dst_width = _node->get_dst_width(), dst_height = _node->get_dst_height();
    const std::vector<float> &angle = _node->angle_values();
    const BoundingBoxCord dest_image{0, 0, static_cast<float>(dst_width), static_cast<float>(dst_height)};
    for (int i = 0; i < (int)in->size(); i++) {
        const Labels labels_buf = in->get_labels_batch()[i];
        const BoundingBoxCords coords_buf = in->get_bb_cords_batch()[i];
        BoundingBoxCords bb_coords;
        Labels bb_labels;
        for (size_t j = 0; j < labels_buf.size(); j++) {
            // meta_node_rotate.cpp:53-77: the four corners through the rotation about the two centres
            const float radian = angle[i] * 3.14159265 / 180;
            float rotate[4];
            rotate[0] = rotate[3] = cos(radian);
            rotate[1] = sin(radian);
            rotate[2] = -1 * rotate[1];
            const float dest_cx = dst_width / 2, dest_cy = dst_height / 2;  // integer halves, as in the reference
            const float src_cx = static_cast<float>(input_roi[i].xywh.w) / 2, src_cy = static_cast<float>(input_roi[i].xywh.h) / 2;
            const float bx = coords_buf[j].l, by = coords_buf[j].t;
            const float bw = coords_buf[j].r - coords_buf[j].l, bh = coords_buf[j].b - coords_buf[j].t;
            const float x1 = (rotate[0] * (bx - src_cx)) + (rotate[1] * (by - src_cy)) + dest_cx;
            const float y1 = (rotate[2] * (bx - src_cx)) + (rotate[3] * (by - src_cy)) + dest_cy;
            const float x2 = (rotate[0] * ((bx + bw) - src_cx)) + (rotate[1] * (by - src_cy)) + dest_cx;
            const float y2 = (rotate[2] * ((bx + bw) - src_cx)) + (rotate[3] * (by - src_cy)) + dest_cy;
            const float x3 = (rotate[0] * (bx - src_cx)) + (rotate[1] * ((by + bh) - src_cy)) + dest_cx;
            const float y3 = (rotate[2] * (bx - src_cx)) + (rotate[3] * ((by + bh) - src_cy)) + dest_cy;
            const float x4 = (rotate[0] * ((bx + bw) - src_cx)) + (rotate[1] * ((by + bh) - src_cy)) + dest_cx;
            const float y4 = (rotate[2] * ((bx + bw) - src_cx)) + (rotate[3] * ((by + bh) - src_cy)) + dest_cy;
            const float min_x = std::min(x1, std::min(x2, std::min(x3, x4))), min_y = std::min(y1, std::min(y2, std::min(y3, y4)));
            BoundingBoxCord box;
            box.l = std::min(0.0f, min_x);
            box.t = std::min(0.0f, min_y);
            box.r = std::max(x1, std::max(x2, std::max(x3, x4)));
            box.b = std::max(y1, std::max(y2, std::max(y3, y4)));
            if (BBoxIntersectionOverUnion(box, dest_image) >= _iou_threshold) {
                box.l = std::max(dest_image.l, box.l);
                box.t = std::max(dest_image.t, box.t);
                box.r = std::min(dest_image.r, box.r);
                box.b = std::min(dest_image.b, box.b);
                bb_coords.push_back(box);
                bb_labels.push_back(labels_buf[j]);
            }
        }
        if (bb_coords.empty()) {
            bb_coords.push_back(dest_image);
            bb_labels.push_back(0);
        }
        out->get_bb_cords_batch()[i] = bb_coords;
        out->get_labels_batch()[i] = bb_labels;
    }
}
