// Bounding-box metadata that follows the images through the hot-path nodes: rocAL's MetaNode classes for
// crop, crop-mirror-normalize, crop-resize, resize, resize-crop-mirror, resize-mirror-normalize, flip and rotate
// (rocAL/include/meta_data/meta_node.h:32-60, rocAL/source/meta_data/meta_node_*.cpp), with the reference's
// arithmetic (fp32, same operation order), its intersection test and its "no box left" fallback boxes.
// Readers are outside the hot path: a batch of boxes is handed in per run, next to the decoded images.
#pragma once
#include <list>
#include <memory>
#include <vector>

#include "nodes.h"

// rocAL/include/meta_data/meta_data.h:36-50
struct BoundingBoxCord {
    float l, t, r, b;
};
typedef std::vector<BoundingBoxCord> BoundingBoxCords;
typedef std::vector<int> Labels;

class MetaDataBatch {
   public:
    explicit MetaDataBatch(size_t batch_size = 0) : _labels(batch_size), _cords(batch_size) {}
    size_t size() const { return _labels.size(); }
    std::vector<Labels> &get_labels_batch() { return _labels; }
    std::vector<BoundingBoxCords> &get_bb_cords_batch() { return _cords; }
    std::shared_ptr<MetaDataBatch> clone(bool copy_contents = true) const {
        return copy_contents ? std::make_shared<MetaDataBatch>(*this) : std::make_shared<MetaDataBatch>(size());
    }

   private:
    std::vector<Labels> _labels;
    std::vector<BoundingBoxCords> _cords;
};
typedef std::shared_ptr<MetaDataBatch> pMetaDataBatch;

class MetaNode {
   public:
    virtual ~MetaNode() = default;
    virtual void update_parameters(pMetaDataBatch input_meta_data, pMetaDataBatch output_meta_data) = 0;
    // meta_node.h:42-60: intersection over the first box's area (over the union when is_iou)
    double BBoxIntersectionOverUnion(const BoundingBoxCord &box1, const BoundingBoxCord &box2, bool is_iou = false) const;
    int _batch_size = 0;
    float _iou_threshold = 0.25;
};

// bounding_box_graph.cpp:24-31: the nodes run in creation order, each on the previous one's output
class BoundingBoxGraph {
   public:
    void process(pMetaDataBatch input_meta_data, pMetaDataBatch output_meta_data);
    std::list<std::shared_ptr<MetaNode>> _meta_nodes;
};

#define RMX_META_NODE(Name, NodeT)                                                                          \
    class Name : public MetaNode {                                                                          \
       public:                                                                                              \
        void update_parameters(pMetaDataBatch input_meta_data, pMetaDataBatch output_meta_data) override;   \
        std::shared_ptr<NodeT> _node = nullptr;                                                             \
    };

RMX_META_NODE(CropMetaNode, CropNode)                                            // meta_node_crop.cpp:30-81
RMX_META_NODE(CropMirrorNormalizeMetaNode, CropMirrorNormalizeNode)              // meta_node_crop_mirror_normalize.cpp:31-87
RMX_META_NODE(CropResizeMetaNode, CropResizeNode)                                // meta_node_crop_resize.cpp:29-86
RMX_META_NODE(ResizeMetaNode, ResizeNode)                                        // meta_node_resize.cpp:24-55
RMX_META_NODE(ResizeCropMirrorMetaNode, ResizeCropMirrorNode)                    // meta_node_resize_crop_mirror.cpp:32-101
RMX_META_NODE(ResizeMirrorNormalizeMetaNode, ResizeMirrorNormalizeNode)          // meta_node_resize_mirror_normalize.cpp:28-86
RMX_META_NODE(FlipMetaNode, FlipNode)                                            // meta_node_flip.cpp:28-60
RMX_META_NODE(RotateMetaNode, RotateNode)                                        // meta_node_rotate.cpp:26-97
#undef RMX_META_NODE
