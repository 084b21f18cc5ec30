// Dependency-free reader for the subset of the ONNX protobuf schema that the
// sparse runtime consumes.  The reference parses with libprotobuf and generated
// classes (src/sparse_onnx.cpp:101-107); neither exists in a ROCm image, so this
// walks the protobuf wire format directly.  Field numbers are those of onnx.proto
// (ModelProto.graph = 7; GraphProto.node = 1, initializer = 5, input = 11,
// output = 12; NodeProto.input = 1, output = 2, op_type = 4, attribute = 5;
// AttributeProto.name = 1, f = 2, i = 3, s = 4, t = 5, floats = 7, ints = 8,
// type = 20; TensorProto.dims = 1, data_type = 2, float_data = 4, int64_data = 7,
// name = 8, raw_data = 9; ValueInfoProto.name = 1, type = 2;
// TypeProto.tensor_type = 1 {elem_type = 1, shape = 2}; TensorShapeProto.dim = 1
// {dim_value = 1, dim_param = 2}).  Unknown fields are skipped.
#pragma once

#include <cstdint>
#include <string>
#include <utility>
#include <vector>

namespace onnxwire {

enum DataType { DT_UNDEFINED = 0, DT_FLOAT = 1, DT_INT32 = 6, DT_INT64 = 7, DT_DOUBLE = 11 };

struct Tensor {
    std::string name;
    std::vector<int64_t> dims;
    int32_t data_type = DT_UNDEFINED;
    std::vector<float> float_data;
    std::vector<int64_t> int64_data;
    std::string raw_data;

    std::size_t numel() const;
    /// Values as fp32 (raw_data first, then float_data, as src/sparse_onnx.cpp:55-78).
    /// Throws std::runtime_error("ONNX tensor has no weight data") when neither is present.
    std::vector<float> floats() const;
};

struct Attribute {
    std::string name;
    int32_t type = 0;
    float f = 0.0f;
    int64_t i = 0;
    std::string s;
    std::vector<float> floats;
    std::vector<int64_t> ints;
};

struct Node {
    std::vector<std::string> input, output;
    std::string name, op_type;
    std::vector<Attribute> attribute;
    const Attribute *find(const std::string &attr_name) const;
};

struct Dimension {
    bool has_value = false;
    int64_t value = 0;
    std::string param;
};

struct ValueInfo {
    std::string name;
    int32_t elem_type = DT_UNDEFINED;
    bool has_shape = false;
    std::vector<Dimension> dims;
};

struct Graph {
    std::string name;
    std::vector<Node> node;
    std::vector<Tensor> initializer;
    std::vector<ValueInfo> input, output;
};

struct Model {
    int64_t ir_version = 0;
    std::string producer_name;
    std::vector<std::pair<std::string, int64_t>> opset_import;
    bool has_graph = false;
    Graph graph;
};

/// Throws std::runtime_error on malformed or truncated input.
Model parse_model(const void *data, std::size_t size);
/// Throws std::runtime_error("Failed to open/parse ONNX file: <path>") as the
/// reference does (src/sparse_onnx.cpp:104-106).
Model load_model(const std::string &path);

} // namespace onnxwire
