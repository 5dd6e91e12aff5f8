// ONNX front door: a reader of the protobuf wire format for the ONNX messages the importer needs, and the
// conversion of a model into the graph IR (the part of src/nnfusion/frontend/onnx_import/{onnx.cpp,
// util/graph_convert.cpp} that the quantized path needs).
#include "nnfusion/frontend/onnx_import/onnx.hpp"

#include "../nnf_datagen.h"
#include "nnfusion/core/operators/generic_op/generic_op.hpp"

#include <cmath>
#include <cstring>
#include <fstream>
#include <iterator>
#include <set>

namespace nnfusion
{
    namespace frontend
    {
        namespace onnx_lite
        {
            namespace
            {
                // one message: a bounded byte range walked field by field
                class Reader
                {
                public:
                    Reader(const uint8_t* p, size_t n)
                        : m_p(p)
                        , m_end(p + n)
                    {
                    }
                    bool done() const { return m_p >= m_end; }
                    uint64_t varint()
                    {
                        uint64_t v = 0;
                        for (int shift = 0; shift < 64; shift += 7)
                        {
                            NNFUSION_CHECK(m_p < m_end) << "onnx: truncated varint";
                            const uint8_t c = *m_p++;
                            v |= (uint64_t)(c & 0x7F) << shift;
                            if (!(c & 0x80))
                                return v;
                        }
                        NNFUSION_CHECK(false) << "onnx: varint longer than 10 bytes";
                        return 0;
                    }
                    // next field: number and wire type
                    void key(uint32_t& field, uint32_t& wire)
                    {
                        const uint64_t k = varint();
                        field = (uint32_t)(k >> 3);
                        wire = (uint32_t)(k & 7);
                    }
                    Reader bytes()
                    {
                        const uint64_t n = varint();
                        NNFUSION_CHECK(n <= (uint64_t)(m_end - m_p)) << "onnx: length-delimited field runs past its message";
                        Reader r(m_p, (size_t)n);
                        m_p += n;
                        return r;
                    }
                    std::string str()
                    {
                        Reader r = bytes();
                        return std::string(reinterpret_cast<const char*>(r.m_p), r.size());
                    }
                    uint32_t fixed32()
                    {
                        NNFUSION_CHECK(m_end - m_p >= 4) << "onnx: truncated 32-bit field";
                        uint32_t v;
                        memcpy(&v, m_p, 4);
                        m_p += 4;
                        return v;
                    }
                    uint64_t fixed64()
                    {
                        NNFUSION_CHECK(m_end - m_p >= 8) << "onnx: truncated 64-bit field";
                        uint64_t v;
                        memcpy(&v, m_p, 8);
                        m_p += 8;
                        return v;
                    }
                    void skip(uint32_t wire)
                    {
                        switch (wire)
                        {
                        case 0: varint(); break;
                        case 1: fixed64(); break;
                        case 2: bytes(); break;
                        case 5: fixed32(); break;
                        default: NNFUSION_CHECK(false) << "onnx: unsupported wire type " << wire;
                        }
                    }
                    const uint8_t* data() const { return m_p; }
                    size_t size() const { return (size_t)(m_end - m_p); }

                private:
                    const uint8_t* m_p;
                    const uint8_t* m_end;
                };

                // repeated scalar field: packed (wire type 2) or one element per key
                template <class T, class F>
                void repeated(Reader& r, uint32_t wire, uint32_t scalar_wire, std::vector<T>& out, F read_one)
                {
                    if (wire == 2)
                    {
                        Reader p = r.bytes();
                        while (!p.done())
                            out.push_back(read_one(p));
                    }
                    else
                    {
                        NNFUSION_CHECK(wire == scalar_wire) << "onnx: unexpected wire type in a repeated field";
                        out.push_back(read_one(r));
                    }
                }
                float as_float(uint32_t bits)
                {
                    float f;
                    memcpy(&f, &bits, 4);
                    return f;
                }
                size_t type_size(int dt)
                {
                    switch (dt)
                    {
                    case UINT8: case INT8: case BOOL: return 1;
                    case UINT16: case INT16: case FLOAT16: return 2;
                    case FLOAT: case INT32: case UINT32: return 4;
                    case INT64: case UINT64: case DOUBLE: return 8;
                    default: return 0;
                    }
                }

                Tensor parse_tensor(Reader r)
                {
                    Tensor t;
                    std::vector<float> float_data;
                    std::vector<int64_t> int32_data, int64_data;
                    std::vector<uint64_t> uint64_data, double_bits;
                    bool raw = false;
                    while (!r.done())
                    {
                        uint32_t f, w;
                        r.key(f, w);
                        switch (f)
                        {
                        case 1: repeated(r, w, 0, t.dims, [](Reader& x) { return (int64_t)x.varint(); }); break;
                        case 2: t.data_type = (int)r.varint(); break;
                        case 4: repeated(r, w, 5, float_data, [](Reader& x) { return as_float(x.fixed32()); }); break;
                        case 5: repeated(r, w, 0, int32_data, [](Reader& x) { return (int64_t)x.varint(); }); break;
                        case 7: repeated(r, w, 0, int64_data, [](Reader& x) { return (int64_t)x.varint(); }); break;
                        case 8: t.name = r.str(); break;
                        case 9:
                        {
                            Reader b = r.bytes();
                            t.bytes.assign(b.data(), b.data() + b.size());
                            raw = true;
                            break;
                        }
                        case 10: repeated(r, w, 1, double_bits, [](Reader& x) { return x.fixed64(); }); break;
                        case 11: repeated(r, w, 0, uint64_data, [](Reader& x) { return x.varint(); }); break;
                        default: r.skip(w);
                        }
                    }
                    if (!raw)
                    {
                        // typed fields: widen / narrow to the tensor's own element type
                        const size_t es = type_size(t.data_type);
                        auto put = [&](const void* p) { t.bytes.insert(t.bytes.end(), (const uint8_t*)p, (const uint8_t*)p + es); };
                        if (t.data_type == FLOAT)
                            for (float v : float_data)
                                put(&v);
                        else if (t.data_type == DOUBLE)
                            for (uint64_t v : double_bits)
                                put(&v);
                        else if (t.data_type == INT64)
                            for (int64_t v : int64_data)
                                put(&v);
                        else if (t.data_type == UINT64 || t.data_type == UINT32)
                            for (uint64_t v : uint64_data)
                                put(&v); // little endian: the low bytes
                        else
                            for (int64_t v : int32_data)
                                put(&v); // int32_data carries INT32, INT16, INT8, UINT16, UINT8, BOOL and FLOAT16 bit patterns
                    }
                    return t;
                }

                Attribute parse_attribute(Reader r)
                {
                    Attribute a;
                    while (!r.done())
                    {
                        uint32_t f, w;
                        r.key(f, w);
                        switch (f)
                        {
                        case 1: a.name = r.str(); break;
                        case 2: a.f = as_float(r.fixed32()); break;
                        case 3: a.i = (int64_t)r.varint(); break;
                        case 4: a.s = r.str(); break;
                        case 5: a.t = parse_tensor(r.bytes()); break;
                        case 7: repeated(r, w, 5, a.floats, [](Reader& x) { return as_float(x.fixed32()); }); break;
                        case 8: repeated(r, w, 0, a.ints, [](Reader& x) { return (int64_t)x.varint(); }); break;
                        case 20: a.type = (int)r.varint(); break;
                        default: r.skip(w);
                        }
                    }
                    return a;
                }

                Node parse_node(Reader r)
                {
                    Node n;
                    while (!r.done())
                    {
                        uint32_t f, w;
                        r.key(f, w);
                        switch (f)
                        {
                        case 1: n.inputs.push_back(r.str()); break;
                        case 2: n.outputs.push_back(r.str()); break;
                        case 3: n.name = r.str(); break;
                        case 4: n.op_type = r.str(); break;
                        case 5:
                        {
                            Attribute a = parse_attribute(r.bytes());
                            n.attributes[a.name] = a;
                            break;
                        }
                        case 7: n.domain = r.str(); break;
                        default: r.skip(w);
                        }
                    }
                    return n;
                }

                ValueInfo parse_value_info(Reader r)
                {
                    ValueInfo v;
                    while (!r.done())
                    {
                        uint32_t f, w;
                        r.key(f, w);
                        if (f == 1)
                            v.name = r.str();
                        else if (f == 2)
                        {
                            Reader type = r.bytes(); // TypeProto
                            while (!type.done())
                            {
                                uint32_t tf, tw;
                                type.key(tf, tw);
                                if (tf != 1)
                                {
                                    type.skip(tw);
                                    continue;
                                }
                                Reader tt = type.bytes(); // TypeProto.Tensor
                                while (!tt.done())
                                {
                                    uint32_t f2, w2;
                                    tt.key(f2, w2);
                                    if (f2 == 1)
                                        v.elem_type = (int)tt.varint();
                                    else if (f2 == 2)
                                    {
                                        Reader shape = tt.bytes(); // TensorShapeProto
                                        while (!shape.done())
                                        {
                                            uint32_t f3, w3;
                                            shape.key(f3, w3);
                                            if (f3 != 1)
                                            {
                                                shape.skip(w3);
                                                continue;
                                            }
                                            Reader dim = shape.bytes();
                                            int64_t value = -1;
                                            std::string param;
                                            while (!dim.done())
                                            {
                                                uint32_t f4, w4;
                                                dim.key(f4, w4);
                                                if (f4 == 1)
                                                    value = (int64_t)dim.varint();
                                                else if (f4 == 2)
                                                    param = dim.str();
                                                else
                                                    dim.skip(w4);
                                            }
                                            v.dims.push_back(value);
                                            v.dim_params.push_back(param);
                                        }
                                    }
                                    else
                                        tt.skip(w2);
                                }
                            }
                        }
                        else
                            r.skip(w);
                    }
                    return v;
                }

                void parse_graph(Reader r, Model& m)
                {
                    while (!r.done())
                    {
                        uint32_t f, w;
                        r.key(f, w);
                        switch (f)
                        {
                        case 1: m.nodes.push_back(parse_node(r.bytes())); break;
                        case 2: m.graph_name = r.str(); break;
                        case 5: m.initializers.push_back(parse_tensor(r.bytes())); break;
                        case 11: m.inputs.push_back(parse_value_info(r.bytes())); break;
                        case 12: m.outputs.push_back(parse_value_info(r.bytes())); break;
                        default: r.skip(w);
                        }
                    }
                }
            } // namespace

            size_t Tensor::element_count() const
            {
                size_t n = 1;
                for (int64_t d : dims)
                    n *= (size_t)d;
                return n;
            }
            int64_t Node::get_int(const std::string& key, int64_t dflt) const
            {
                auto it = attributes.find(key);
                return it == attributes.end() ? dflt : it->second.i;
            }
            float Node::get_float(const std::string& key, float dflt) const
            {
                auto it = attributes.find(key);
                return it == attributes.end() ? dflt : it->second.f;
            }

            Model parse_model(const std::vector<uint8_t>& file)
            {
                Model m;
                Reader r(file.data(), file.size());
                while (!r.done())
                {
                    uint32_t f, w;
                    r.key(f, w);
                    switch (f)
                    {
                    case 1: m.ir_version = (int64_t)r.varint(); break;
                    case 2: m.producer_name = r.str(); break;
                    case 7: parse_graph(r.bytes(), m); break;
                    case 8:
                    {
                        Reader o = r.bytes(); // OperatorSetIdProto
                        std::string domain;
                        int64_t version = 0;
                        while (!o.done())
                        {
                            uint32_t f2, w2;
                            o.key(f2, w2);
                            if (f2 == 1)
                                domain = o.str();
                            else if (f2 == 2)
                                version = (int64_t)o.varint();
                            else
                                o.skip(w2);
                        }
                        m.opset[domain] = version;
                        break;
                    }
                    default: r.skip(w);
                    }
                }
                return m;
            }

            Model parse_model_file(const std::string& path)
            {
                std::ifstream f(path, std::ios::binary);
                NNFUSION_CHECK(f.is_open()) << "onnx: cannot open " << path;
                std::vector<uint8_t> bytes((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
                return parse_model(bytes);
            }
        } // namespace onnx_lite

        namespace
        {
            using namespace onnx_lite;

            const element::Type& element_type_of(int dt)
            {
                switch (dt)
                {
                case FLOAT: return element::f32;
                case FLOAT16: return element::f16;
                case DOUBLE: return element::f64;
                case UINT8: return element::u8;
                case INT8: return element::i8;
                case INT32: return element::i32;
                case INT64: return element::i64;
                case BOOL: return element::boolean;
                default: NNFUSION_CHECK(false) << "onnx: unsupported tensor element type " << dt; return element::dynamic;
                }
            }

            size_t type_bytes(int dt) { return dt == FLOAT16 ? 2 : dt == FLOAT ? 4 : 1; }

            // fp32 -> fp16 bits, round to nearest even (scales stored as fp32 in a model)
            uint16_t float_to_half_bits(float f)
            {
                return nnf_f32_to_f16_bits(f);
            }
        } // namespace

        std::shared_ptr<graph::Graph> load_onnx_model(const std::string& path,
                                                      const std::unordered_map<std::string, size_t>& dim_params)
        {
            const Model model = parse_model_file(path);
            auto g = std::make_shared<graph::Graph>();
            std::map<std::string, std::shared_ptr<graph::GNode>> value; // ONNX value name -> producing node
            std::map<std::string, const Tensor*> init;
            for (auto& t : model.initializers)
                init[t.name] = &t;

            auto add_constant = [&](const Tensor& t, const std::string& name) {
                const element::Type& et = element_type_of(t.data_type);
                Shape shape;
                for (int64_t d : t.dims)
                    shape.push_back((size_t)d);
                NNFUSION_CHECK(t.bytes.size() == shape_size(shape) * et.size())
                    << "onnx: tensor " << name << " carries " << t.bytes.size() << " bytes for " << shape_size(shape) << " elements";
                value[name] = g->add_node_and_edge(std::make_shared<op::Constant>(et, shape, t.bytes.data()), graph::GNodeVector{});
            };
            // graph inputs that are not initializers are the parameters, in file order
            for (auto& in : model.inputs)
            {
                if (init.count(in.name))
                    continue;
                Shape shape;
                for (size_t i = 0; i < in.dims.size(); ++i)
                {
                    int64_t d = in.dims[i];
                    if (d < 0)
                    {
                        auto it = dim_params.find(in.dim_params[i]);
                        NNFUSION_CHECK(it != dim_params.end()) << "onnx: no value for the symbolic dimension '" << in.dim_params[i]
                                                               << "' of input " << in.name;
                        d = (int64_t)it->second;
                    }
                    shape.push_back((size_t)d);
                }
                value[in.name] = g->add_node_and_edge(std::make_shared<op::Parameter>(element_type_of(in.elem_type), shape),
                                                      graph::GNodeVector{});
            }
            auto input_of = [&](const Node& n, size_t i) -> std::shared_ptr<graph::GNode> {
                NNFUSION_CHECK(i < n.inputs.size()) << "onnx: " << n.op_type << " " << n.name << " has no input " << i;
                const std::string& name = n.inputs[i];
                auto it = value.find(name);
                if (it != value.end())
                    return it->second;
                auto ti = init.find(name);
                NNFUSION_CHECK(ti != init.end()) << "onnx: " << n.op_type << " " << n.name << " reads undefined value " << name;
                add_constant(*ti->second, name); // initializers become constants where they are first used
                return value[name];
            };
            auto has_input = [](const Node& n, size_t i) { return i < n.inputs.size() && !n.inputs[i].empty(); };
            auto generic = [&](const Node& n, const std::string& type, const graph::GNodeVector& in, const std::string& cfg = "") {
                auto config = cfg.empty() ? op::OpConfig::any() : op::OpConfig::any::parse(cfg);
                const std::string name = n.name.empty() ? n.outputs.at(0) : n.name;
                return g->add_node_and_edge(std::make_shared<op::GenericOp>(name, type, config), in);
            };

            // input i of node n as an fp16 row of `len` values: a value of the graph, or an initializer (fp16, or fp32 rounded)
            auto half_row = [&](const Node& n, size_t i, size_t len) -> std::shared_ptr<graph::GNode> {
                auto ti = init.find(n.inputs[i]);
                if (ti == init.end() || ti->second->data_type == FLOAT16)
                {
                    auto v = input_of(n, i);
                    NNFUSION_CHECK(shape_size(v->get_output_shape(0)) == len && v->get_output_element_type(0) == element::f16)
                        << "onnx: " << n.op_type << " " << n.name << ": input " << i << " must be fp16 [" << len << "]";
                    return v;
                }
                const Tensor& t = *ti->second;
                NNFUSION_CHECK(t.data_type == FLOAT && t.bytes.size() == len * 4)
                    << "onnx: " << n.op_type << " " << n.name << ": input " << i << " must be fp16 or fp32 [" << len << "]";
                std::vector<uint16_t> h(len);
                for (size_t j = 0; j < len; ++j)
                {
                    float f;
                    memcpy(&f, t.bytes.data() + 4 * j, 4);
                    h[j] = float_to_half_bits(f);
                }
                return g->add_node_and_edge(std::make_shared<op::Constant>(element::f16, Shape{len}, h.data()), graph::GNodeVector{});
            };
            // values produced by a DequantizeLinear of weights [K, N]: held as the Dequantize of the weights in the
            // layout of the kernels, [N, K] -- a MatMul that reads one becomes a Dot with transpose_B
            std::set<std::string> transposed_weights;
            // element (r, c) of a 2-D initializer of 4- or 8-bit integers, as an unsigned value (signed types: + 2^(bits-1))
            auto small_int_at = [](const Tensor& t, int bits, bool is_signed, size_t cols, size_t r, size_t c) -> int {
                const size_t i = r * cols + c;
                int v;
                if (bits == 8)
                    v = is_signed ? (int)(int8_t)t.bytes[i] + 128 : (int)t.bytes[i];
                else
                {
                    const int nib = (t.bytes[i >> 1] >> (4 * (i & 1))) & 0xF;
                    v = is_signed ? ((nib ^ 8) - 8) + 8 : nib; // sign-extend, then shift the range to 0 .. 15
                }
                return v;
            };

            for (auto& n : model.nodes) // ONNX keeps nodes in topological order
            {
                NNFUSION_CHECK(!n.outputs.empty()) << "onnx: node without outputs";
                std::shared_ptr<graph::GNode> out;
                if (n.op_type == "Constant")
                {
                    auto it = n.attributes.find("value");
                    NNFUSION_CHECK(it != n.attributes.end()) << "onnx: Constant without a value tensor";
                    add_constant(it->second.t, n.outputs[0]);
                    continue;
                }
                else if (n.op_type == "MatMulNBits")
                {
                    // A [.., K]; B u8 [N, K/block, block*bits/8] (4 bits: two values per byte, low nibble first);
                    // scales [N * K/block]; optional zero_points u8 [N, ceil(K/block * bits / 8)], one per block
                    // (4-bit ones two per byte along the blocks of a row, even block in the low nibble); without them the
                    // zero point is 2^(bits-1)
                    const int64_t K = n.get_int("K", 0), N = n.get_int("N", 0);
                    const int64_t bits = n.get_int("bits", 4), block = n.get_int("block_size", 0);
                    NNFUSION_CHECK((bits == 4 || bits == 8) && (block == 32 || block == 64 || block == 128) && K > 0 && N > 0 &&
                                   K % block == 0)
                        << "onnx: MatMulNBits " << n.name
                        << ": bits = 4 or 8 and block_size = 32, 64 or 128 (K a multiple of it) are supported";
                    NNFUSION_CHECK(!has_input(n, 4)) << "onnx: MatMulNBits with g_idx is not supported";
                    auto wi = init.find(n.inputs.at(1));
                    auto si = init.find(n.inputs.at(2));
                    NNFUSION_CHECK(wi != init.end() && si != init.end()) << "onnx: MatMulNBits weights and scales must be initializers";
                    const Tensor& wt = *wi->second;
                    NNFUSION_CHECK(wt.data_type == UINT8 && wt.bytes.size() == (size_t)(N * K * bits / 8))
                        << "onnx: MatMulNBits B must be uint8 with N*K*bits/8 bytes";
                    int zp = 1 << (bits - 1);
                    std::shared_ptr<graph::GNode> zps; // set when the zero points differ between blocks
                    if (has_input(n, 3))
                    {
                        const int64_t blocks = K / block, z_stride = (blocks * bits + 7) / 8;
                        auto zi = init.find(n.inputs[3]);
                        NNFUSION_CHECK(zi != init.end() && zi->second->data_type == UINT8 &&
                                       zi->second->bytes.size() == (size_t)(N * z_stride))
                            << "onnx: MatMulNBits zero points must be a packed uint8 initializer of N * ceil(K/block_size*bits/8) bytes";
                        const std::vector<uint8_t>& z = zi->second->bytes;
                        auto at = [&](int64_t r, int64_t b) -> int {
                            if (bits == 8)
                                return z[(size_t)(r * z_stride + b)];
                            const uint8_t byte = z[(size_t)(r * z_stride + b / 2)];
                            return (b & 1) ? (byte >> 4) : (byte & 0xF);
                        };
                        zp = at(0, 0);
                        bool uniform = true;
                        for (int64_t r = 0; r < N && uniform; ++r)
                            for (int64_t b = 0; b < blocks; ++b)
                                if (at(r, b) != zp)
                                {
                                    uniform = false;
                                    break;
                                }
                        // one value everywhere is the scalar attribute (the specialised kernels take it); otherwise the
                        // tensor travels with the node
                        if (!uniform)
                            zps = g->add_node_and_edge(
                                std::make_shared<op::Constant>(element::u8, Shape{(size_t)N, (size_t)z_stride}, z.data()),
                                graph::GNodeVector{});
                    }
                    auto wq = g->add_node_and_edge(
                        std::make_shared<op::Constant>(element::u8, Shape{(size_t)N, (size_t)(K * bits / 8)}, wt.bytes.data()), graph::GNodeVector{});
                    const Tensor& st = *si->second;
                    const size_t n_scales = (size_t)(N * (K / block));
                    std::vector<uint16_t> sc(n_scales);
                    if (st.data_type == FLOAT16)
                    {
                        NNFUSION_CHECK(st.bytes.size() == n_scales * 2) << "onnx: MatMulNBits scales: wrong size";
                        memcpy(sc.data(), st.bytes.data(), n_scales * 2);
                    }
                    else
                    {
                        NNFUSION_CHECK(st.data_type == FLOAT && st.bytes.size() == n_scales * 4) << "onnx: MatMulNBits scales must be fp16 or fp32";
                        for (size_t i = 0; i < n_scales; ++i)
                        {
                            float f;
                            memcpy(&f, st.bytes.data() + 4 * i, 4);
                            sc[i] = float_to_half_bits(f);
                        }
                    }
                    auto s = g->add_node_and_edge(
                        std::make_shared<op::Constant>(element::f16, Shape{(size_t)N, (size_t)(K / block)}, sc.data()), graph::GNodeVector{});
                    // input 5: a bias [N], added to every row: the product's own epilogue
                    std::shared_ptr<graph::GNode> bias;
                    if (has_input(n, 5))
                        bias = half_row(n, 5, (size_t)N);
                    std::string attrs = "{\"bits\": " + std::to_string(bits) + ", \"group_size\": " + std::to_string(block) +
                                        ", \"zero_point\": " + std::to_string(zps ? 0 : zp) +
                                        ", \"has_zero_points\": " + (zps ? "true" : "false") +
                                        ", \"has_bias\": " + (bias ? "true" : "false") + "}";
                    graph::GNodeVector ins = {input_of(n, 0), wq, s};
                    if (zps)
                        ins.push_back(zps);
                    if (bias)
                        ins.push_back(bias);
                    out = generic(n, "QuantDot", ins, attrs);
                }
                else if (n.op_type == "DequantizeLinear")
                {
                    // Blocked dequantisation of a weight matrix W [K, N] (the B operand of a MatMul): axis = 0,
                    // block_size = 32 / 64 / 128 along K, x_scale [K / block, N], optional x_zero_point of x's type and
                    // x_scale's shape; y = (x - zero point) * scale.  4-bit types two per byte, first element low.  Signed
                    // types are shifted to unsigned ones with the zero point (q + 2^(bits-1), z + 2^(bits-1)).
                    auto xi = init.find(n.inputs.at(0));
                    auto si = init.find(n.inputs.at(1));
                    NNFUSION_CHECK(xi != init.end() && si != init.end())
                        << "onnx: DequantizeLinear " << n.name << ": only quantized weights (initializers) are supported";
                    const Tensor& xt = *xi->second;
                    const Tensor& st = *si->second;
                    const int dt = xt.data_type;
                    NNFUSION_CHECK(dt == UINT8 || dt == INT8 || dt == UINT4 || dt == INT4)
                        << "onnx: DequantizeLinear " << n.name << ": weights must be (u)int8 or (u)int4";
                    const int bits = (dt == UINT8 || dt == INT8) ? 8 : 4;
                    const bool is_signed = dt == INT8 || dt == INT4;
                    const int64_t block = n.get_int("block_size", 0), axis = n.get_int("axis", 1);
                    NNFUSION_CHECK(xt.dims.size() == 2 && (axis == 0 || axis == -2) && (block == 32 || block == 64 || block == 128) &&
                                   xt.dims[0] % block == 0)
                        << "onnx: DequantizeLinear " << n.name
                        << ": a weight matrix [K, N] with axis = 0 and block_size = 32, 64 or 128 (K a multiple of it) is supported";
                    const size_t K = (size_t)xt.dims[0], N = (size_t)xt.dims[1], G = K / (size_t)block;
                    NNFUSION_CHECK(xt.bytes.size() == (K * N * bits + 7) / 8) << "onnx: DequantizeLinear " << n.name << ": wrong data size";
                    NNFUSION_CHECK(st.dims.size() == 2 && (size_t)st.dims[0] == G && (size_t)st.dims[1] == N &&
                                   (st.data_type == FLOAT16 || st.data_type == FLOAT) && st.bytes.size() == G * N * type_bytes(st.data_type))
                        << "onnx: DequantizeLinear " << n.name << ": scales must be fp16 or fp32 [K / block_size, N]";
                    // weights -> [N, K * bits / 8], packed along K (4 bits: even k in the low nibble)
                    std::vector<uint8_t> wq(N * K * bits / 8, 0);
                    for (size_t k = 0; k < K; ++k)
                        for (size_t c = 0; c < N; ++c)
                        {
                            const int v = small_int_at(xt, bits, is_signed, N, k, c);
                            if (bits == 8)
                                wq[c * K + k] = (uint8_t)v;
                            else
                                wq[c * (K / 2) + k / 2] |= (uint8_t)(v << (4 * (k & 1)));
                        }
                    // scales -> fp16 [N, K / block]
                    std::vector<uint16_t> sc(N * G);
                    for (size_t b = 0; b < G; ++b)
                        for (size_t c = 0; c < N; ++c)
                        {
                            if (st.data_type == FLOAT16)
                                memcpy(&sc[c * G + b], st.bytes.data() + 2 * (b * N + c), 2);
                            else
                            {
                                float f;
                                memcpy(&f, st.bytes.data() + 4 * (b * N + c), 4);
                                sc[c * G + b] = float_to_half_bits(f);
                            }
                        }
                    // zero points: one value everywhere is the scalar attribute, otherwise u8 [N, ceil(G * bits / 8)]
                    int zp = is_signed ? (1 << (bits - 1)) : 0;
                    std::vector<uint8_t> zq;
                    bool uniform = true;
                    if (has_input(n, 2))
                    {
                        auto zi = init.find(n.inputs[2]);
                        NNFUSION_CHECK(zi != init.end() && zi->second->data_type == dt && zi->second->dims.size() == 2 &&
                                       (size_t)zi->second->dims[0] == G && (size_t)zi->second->dims[1] == N &&
                                       zi->second->bytes.size() == (G * N * bits + 7) / 8)
                            << "onnx: DequantizeLinear " << n.name << ": zero points must have the weights' type and the scales' shape";
                        const Tensor& zt = *zi->second;
                        const size_t z_stride = (G * bits + 7) / 8;
                        zq.assign(N * z_stride, 0);
                        zp = small_int_at(zt, bits, is_signed, N, 0, 0);
                        for (size_t b = 0; b < G; ++b)
                            for (size_t c = 0; c < N; ++c)
                            {
                                const int v = small_int_at(zt, bits, is_signed, N, b, c);
                                uniform = uniform && v == zp;
                                if (bits == 8)
                                    zq[c * z_stride + b] = (uint8_t)v;
                                else
                                    zq[c * z_stride + b / 2] |= (uint8_t)(v << (4 * (b & 1)));
                            }
                    }
                    graph::GNodeVector ins = {
                        g->add_node_and_edge(std::make_shared<op::Constant>(element::u8, Shape{N, K * bits / 8}, wq.data()), graph::GNodeVector{}),
                        g->add_node_and_edge(std::make_shared<op::Constant>(element::f16, Shape{N, G}, sc.data()), graph::GNodeVector{})};
                    const bool has_z = !zq.empty() && !uniform;
                    if (has_z)
                        ins.push_back(g->add_node_and_edge(
                            std::make_shared<op::Constant>(element::u8, Shape{N, (G * bits + 7) / 8}, zq.data()), graph::GNodeVector{}));
                    const std::string attrs = "{\"bits\": " + std::to_string(bits) + ", \"group_size\": " + std::to_string(block) +
                                              ", \"zero_point\": " + std::to_string(has_z ? 0 : zp) +
                                              ", \"has_zero_points\": " + (has_z ? "true" : "false") + "}";
                    out = generic(n, "Dequantize", ins, attrs);
                    transposed_weights.insert(n.outputs[0]);
                }
                else if (n.op_type == "MatMul")
                {
                    // (a Dot of two fp16 values has no kernel in this library: the fold into QuantDot is what makes it run)
                    const bool tb = transposed_weights.count(n.inputs.at(1)) != 0;
                    out = generic(n, "Dot", {input_of(n, 0), input_of(n, 1)}, std::string("{\"transpose_B\": ") + (tb ? "true" : "false") + "}");
                }
                else if (n.op_type == "SimplifiedLayerNormalization" || n.op_type == "RMSNormalization")
                {
                    const int64_t axis = n.get_int("axis", -1);
                    auto x = input_of(n, 0);
                    NNFUSION_CHECK(axis == -1 || axis == (int64_t)x->get_output_shape(0).size() - 1)
                        << "onnx: " << n.op_type << " over an axis other than the last is not supported";
                    char eps[64];
                    snprintf(eps, sizeof(eps), "{\"eps\": %.9g}", (double)n.get_float("epsilon", 1e-5f));
                    out = generic(n, "RMSNorm", {x, input_of(n, 1)}, eps);
                }
                else if (n.op_type == "Sigmoid")
                    out = generic(n, "Sigmoid", {input_of(n, 0)});
                else if (n.op_type == "Mul")
                    out = generic(n, "Multiply", {input_of(n, 0), input_of(n, 1)});
                else if (n.op_type == "Add")
                    out = generic(n, "Add", {input_of(n, 0), input_of(n, 1)});
                else
                    NNFUSION_CHECK(false) << "onnx: unsupported operator " << (n.domain.empty() ? "" : n.domain + "::") << n.op_type;
                value[n.outputs[0]] = out;
            }
            for (auto& o : model.outputs)
            {
                auto it = value.find(o.name);
                NNFUSION_CHECK(it != value.end()) << "onnx: graph output " << o.name << " is not produced";
                g->add_node_and_edge(std::make_shared<op::Result>(), {it->second});
            }
            return g;
        }
    } // namespace frontend
} // namespace nnfusion
