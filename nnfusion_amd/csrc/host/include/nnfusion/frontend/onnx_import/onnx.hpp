// ONNX front door for the quantized path: load_onnx_model() with the signature of the reference's importer
// (src/nnfusion/frontend/onnx_import/onnx.hpp:33-37), restricted to the operators this build has kernels or
// fusion patterns for:
//   com.microsoft::MatMulNBits (bits = 4, block_size = 128, no per-block zero points other than a uniform one)
//                                                           -> QuantDot
//   SimplifiedLayerNormalization / RMSNormalization (last axis) -> RMSNorm
//   Sigmoid, Mul, Add                                       -> Sigmoid, Multiply, Add
// Graph inputs become Parameters, initializers and Constant nodes become Constants, graph outputs Results.
// An unsupported operator raises, as in the reference (onnx_import/util/graph_convert.cpp).
//
// The reference links protobuf and the generated onnx.pb.h; neither exists in this image, so the file is read
// with a small reader of the protobuf wire format (varint / 64-bit / length-delimited / 32-bit fields) and the
// handful of ONNX messages the importer needs (field numbers of onnx.proto3: ModelProto, GraphProto, NodeProto,
// AttributeProto, TensorProto, ValueInfoProto, TypeProto, TensorShapeProto).
#pragma once

#include "nnfusion/core/graph/gnode.hpp"

#include <map>
#include <string>
#include <unordered_map>
#include <vector>

namespace nnfusion
{
    namespace frontend
    {
        namespace onnx_lite
        {
            // TensorProto.DataType values used here
            enum DataType
            {
                UNDEFINED = 0, FLOAT = 1, UINT8 = 2, INT8 = 3, UINT16 = 4, INT16 = 5, INT32 = 6, INT64 = 7,
                STRING = 8, BOOL = 9, FLOAT16 = 10, DOUBLE = 11, UINT32 = 12, UINT64 = 13,
                UINT4 = 21, INT4 = 22 // two per byte in raw_data, the first element in the low nibble
            };
            struct Tensor
            {
                std::string name;
                std::vector<int64_t> dims;
                int data_type = UNDEFINED;
                // the element bytes in the tensor's own type, whichever field carried them
                // (raw_data, float_data, int32_data, int64_data, double_data, uint64_data)
                std::vector<uint8_t> bytes;
                size_t element_count() const;
            };
            struct Attribute
            {
                std::string name;
                int type = 0; // AttributeProto.AttributeType: 1 FLOAT, 2 INT, 3 STRING, 4 TENSOR, 6 FLOATS, 7 INTS
                float f = 0.f;
                int64_t i = 0;
                std::string s;
                Tensor t;
                std::vector<float> floats;
                std::vector<int64_t> ints;
            };
            struct Node
            {
                std::string name, op_type, domain;
                std::vector<std::string> inputs, outputs;
                std::map<std::string, Attribute> attributes;
                int64_t get_int(const std::string& key, int64_t dflt) const;
                float get_float(const std::string& key, float dflt) const;
            };
            struct ValueInfo
            {
                std::string name;
                int elem_type = UNDEFINED;
                std::vector<int64_t> dims;           // -1 where the dimension is symbolic
                std::vector<std::string> dim_params; // the symbol's name there, else empty
            };
            struct Model
            {
                int64_t ir_version = 0;
                std::string producer_name, graph_name;
                std::map<std::string, int64_t> opset; // domain -> version
                std::vector<Node> nodes;
                std::vector<Tensor> initializers;
                std::vector<ValueInfo> inputs, outputs;
            };
            // throws nnfusion::CheckError on malformed input
            Model parse_model(const std::vector<uint8_t>& file);
            Model parse_model_file(const std::string& path);
        } // namespace onnx_lite

        // Convert an ONNX model to a graph.  dim_params: values for symbolic dimensions of the graph inputs.
        std::shared_ptr<nnfusion::graph::Graph>
            load_onnx_model(const std::string& path, const std::unordered_map<std::string, size_t>& dim_params = {});
    } // namespace frontend
} // namespace nnfusion
