// The two opaque handles of include/berth_exl3_reader.h, shared by the translation units
// of libberth_exl3_reader.so (the reader's C interface and the planner's).
#pragma once

#include "exl3_checkpoint.hpp"

#include <vector>

using berth::exl3::Checkpoint;
using berth::exl3::LayerType;
using berth::exl3::ModelConfig;
using berth::exl3::TensorInfo;

struct berth_ckpt_config {
    ModelConfig cfg;
    std::vector<int> kinds;
    std::vector<const char*> names;
    void index()
    {
        kinds.clear();
        names.clear();
        for (const LayerType& t : cfg.layer_types) {
            kinds.push_back((int)t.kind);
            names.push_back(t.name.c_str());
        }
    }
};

struct berth_ckpt {
    Checkpoint ckpt;
    berth_ckpt_config config;
    std::vector<const TensorInfo*> tensors;   // name order
};
