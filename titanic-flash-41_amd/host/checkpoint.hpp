// Header-first, read-only checkpoint loading for the layer's operands: the safetensors shard scan of the reference
// (src/checkpoint.rs:104-215: index + shard headers, never anything executable), the tensor names, dtypes and shapes it
// requires for one FFN layer (src/layout.rs:247-275), and the host-side assembly of the operands in the order the weight
// atlas keeps them (src/weights.rs:276-356: experts in numeric order, up (w3) before gate (w1) in W13; shared expert gate
// (w1) before up (w3), src/blockscaled.rs:132-133), with the expert scale bytes held to the lossless range (<= 247,
// src/weights.rs:538-542).
#pragma once
#include "../../include/titanic_moe.h"
#include <cstdint>
#include <map>
#include <string>
#include <vector>

namespace tf {

struct CheckpointTensor {
    std::string file, dtype;          // dtype as the header spells it: F32, BF16, F8_E4M3, F8_E8M0, I8
    std::vector<uint64_t> shape;
    uint64_t begin = 0, end = 0;      // data_offsets, relative to the shard's data start
    uint64_t bytes() const { return end - begin; }
};
struct CheckpointShard { uint64_t size = 0, data_start = 0; };

class Checkpoint {
public:
    static Checkpoint scan(const std::string& root);                                             // :108-176
    const CheckpointTensor& tensor(const std::string& name) const;
    // layout.rs `require`: the tensor exists with this dtype and shape
    void require(const std::string& name, const std::string& dtype, const std::vector<uint64_t>& shape) const;
    std::vector<uint8_t> read(const std::string& name) const;
    size_t tensors() const { return tensors_.size(); }
    size_t shards() const { return files_.size(); }
private:
    void validate() const;                                                                        // :177-215
    std::string root_;
    std::map<std::string, CheckpointShard> files_;
    std::map<std::string, CheckpointTensor> tensors_;
};

// One layer's operands on the host, canonical layout (what tf::Weights::Host points at).
struct LayerOperandsHost {
    std::vector<uint16_t> gate_w;
    std::vector<float> bias, bias_alt;
    std::vector<uint8_t> w13, s13, w2, s2, sh_w13, sh_s13, sh_w2, sh_s2;
};
// What the loader requires of a checkpoint for one layer, in the order it checks it (src/layout.rs:247-275): every tensor's
// name, dtype as the header spells it, and shape.  load_ffn_layer requires exactly these and reads nothing else.
struct TensorContract { std::string name, dtype; std::vector<uint64_t> shape; };
std::vector<TensorContract> ffn_layer_contract(const std::string& prefix, const ca_geometry& g);
// prefix: the layer's name prefix in the checkpoint ("layers.7"): tensors "<prefix>.ffn.experts.<e>.w1.weight" ...
LayerOperandsHost load_ffn_layer(const Checkpoint& checkpoint, const std::string& prefix, const ca_geometry& g);

}  // namespace tf
