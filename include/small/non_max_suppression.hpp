// Bounding boxes, detections and greedy per-class non-maximum suppression for the YOLO heads (host code;
// same types, member names and results as the reference's include/small/non_max_suppression.hpp:32-156).
#pragma once

#include <algorithm>
#include <cstddef>
#include <ostream>
#include <vector>

namespace small
{

struct BoundingBox
{
    float x, y;   // centre
    float w, h;   // extents

    // length of the overlap of two centred intervals (negative when they are apart)
    static float overlap(float x1, float w1, float x2, float w2)
    {
        const float left = std::max(x1 - w1 / 2, x2 - w2 / 2);
        const float right = std::min(x1 + w1 / 2, x2 + w2 / 2);
        return right - left;
    }

    float iou(BoundingBox const &other) const
    {
        const float wo = overlap(x, w, other.x, other.w);
        const float ho = overlap(y, h, other.y, other.h);
        const float inter = (wo < 0.f || ho < 0.f) ? 0.f : wo * ho;
        return inter / (w * h + other.w * other.h - inter);
    }
};

inline std::ostream &operator<<(std::ostream &os, BoundingBox const &b)
{
    return os << "center(" << b.x << "," << b.y << "),size(" << b.w << "," << b.h << ")";
}

struct Detection
{
    BoundingBox bbox;
    float objectness;    // objectness confidence
    float class_score;   // class confidence
    size_t class_id;
};

inline std::ostream &operator<<(std::ostream &os, Detection const &d)
{
    return os << "[" << d.bbox << ",objectness=" << d.objectness << ",class_id=" << d.class_id
              << ",p(class)=" << d.class_score << ",prob=" << (d.class_score * d.objectness) << "]";
}

// Highest objectness first; a kept detection removes every later one of its class whose IoU with it reaches
// the threshold.  std::sort, as in the reference: the order of equal objectness values is unspecified there too.
inline std::vector<Detection> basic_nms(std::vector<Detection> predictions, float iou_threshold)
{
    std::sort(predictions.begin(), predictions.end(),
              [](Detection const &a, Detection const &b) { return a.objectness > b.objectness; });
    std::vector<Detection> keep;
    std::vector<char> dead(predictions.size(), 0);
    for (size_t i = 0; i < predictions.size(); ++i)
    {
        if (dead[i]) continue;
        keep.push_back(predictions[i]);
        for (size_t j = i + 1; j < predictions.size(); ++j)
            if (!dead[j] && predictions[j].class_id == predictions[i].class_id &&
                !(predictions[i].bbox.iou(predictions[j].bbox) < iou_threshold))
                dead[j] = 1;
    }
    return keep;
}

} // namespace small
