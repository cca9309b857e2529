#include "SOFIE_HIP/RModelParser_ONNX.hxx"
#include "SOFIE_HIP/operators/OperatorList.hxx"

#include <fstream>
#include <iostream>
#include <iterator>
#include <limits>
#include <map>

namespace SOFIE_HIP {
namespace {

struct Slice {
   const uint8_t *p = nullptr;
   size_t n = 0;
};

struct Field {
   uint32_t no;
   uint32_t wt;
   uint64_t v;   // varint or fixed value
   Slice bytes;  // length-delimited payload
};

class Reader {
public:
   explicit Reader(Slice s) : fP(s.p), fEnd(s.p + s.n) {}
   bool Next(Field &f)
   {
      if (fP >= fEnd)
         return false;
      uint64_t key = Varint();
      f.no = (uint32_t)(key >> 3);
      f.wt = (uint32_t)(key & 7);
      f.v = 0;
      f.bytes = Slice{};
      switch (f.wt) {
      case 0: f.v = Varint(); break;
      case 1: f.v = Fixed(8); break;
      case 5: f.v = Fixed(4); break;
      case 2: {
         uint64_t len = Varint();
         if (len > (uint64_t)(fEnd - fP))
            throw std::runtime_error("SOFIE ONNX parser: truncated file");
         f.bytes = Slice{fP, (size_t)len};
         fP += len;
      } break;
      default: throw std::runtime_error("SOFIE ONNX parser: unsupported wire type");
      }
      return true;
   }

private:
   uint64_t Varint()
   {
      uint64_t r = 0;
      int shift = 0;
      while (true) {
         if (fP >= fEnd)
            throw std::runtime_error("SOFIE ONNX parser: truncated varint");
         uint8_t b = *fP++;
         if (shift > 63)
            throw std::runtime_error("SOFIE ONNX parser: varint longer than 10 bytes");
         r |= (uint64_t)(b & 0x7f) << shift;
         if (!(b & 0x80))
            return r;
         shift += 7;
      }
   }
   uint64_t Fixed(int n)
   {
      if (fEnd - fP < n)
         throw std::runtime_error("SOFIE ONNX parser: truncated file");
      uint64_t r = 0;
      for (int i = 0; i < n; ++i)
         r |= (uint64_t)fP[i] << (8 * i);
      fP += n;
      return r;
   }
   const uint8_t *fP, *fEnd;
};

std::string Str(Slice s) { return s.p ? std::string((const char *)s.p, s.n) : std::string(); }
// text of a string / bytes field; a field of that number written with another wire type is a malformed file
std::string Str(const Field &f)
{
   if (f.wt != 2)
      throw std::runtime_error("SOFIE ONNX parser: field " + std::to_string(f.no) + " should be length-delimited");
   return Str(f.bytes);
}

std::vector<int64_t> PackedInts(const Field &f)
{
   std::vector<int64_t> out;
   if (f.wt == 0) {
      out.push_back((int64_t)f.v);
      return out;
   }
   if (f.wt != 2)
      throw std::runtime_error("SOFIE ONNX parser: repeated integer field " + std::to_string(f.no) + " has wire type " + std::to_string(f.wt));
   // a packed field is a sequence of bare varints, each at most 10 bytes long
   const uint8_t *p = f.bytes.p, *e = f.bytes.p + f.bytes.n;
   while (p < e) {
      uint64_t v = 0;
      int shift = 0;
      for (;;) {
         if (p >= e)
            throw std::runtime_error("SOFIE ONNX parser: truncated varint in a packed field");
         if (shift > 63)
            throw std::runtime_error("SOFIE ONNX parser: varint longer than 10 bytes");
         const uint8_t b = *p++;
         v |= (uint64_t)(b & 0x7f) << shift;
         if (!(b & 0x80))
            break;
         shift += 7;
      }
      out.push_back((int64_t)v);
   }
   return out;
}

// repeated float: packed (length-delimited, 4 bytes each) or one fixed32 per occurrence
void AppendFloats(const Field &f, std::vector<float> &out)
{
   if (f.wt == 5) {
      float v;
      const uint32_t bits = (uint32_t)f.v;
      std::memcpy(&v, &bits, 4);
      out.push_back(v);
      return;
   }
   if (f.wt != 2 || f.bytes.n % 4 != 0)
      throw std::runtime_error("SOFIE ONNX parser: repeated float field " + std::to_string(f.no) + " is malformed");
   for (size_t i = 0; i + 4 <= f.bytes.n; i += 4) {
      float v;
      std::memcpy(&v, f.bytes.p + i, 4);
      out.push_back(v);
   }
}

float AsFloat(uint32_t bits)
{
   float f;
   std::memcpy(&f, &bits, 4);
   return f;
}

struct Tensor {
   std::string name;
   int dtype = 1;
   std::vector<size_t> dims;
   std::vector<uint8_t> raw;        // raw_data
   std::vector<float> floats;       // float_data
   std::vector<int64_t> ints;       // int32_data / int64_data
};

Tensor ParseTensor(Slice s)
{
   Tensor t;
   Reader r(s);
   Field f;
   while (r.Next(f)) {
      switch (f.no) {
      case 1:
         for (auto d : PackedInts(f))
            t.dims.push_back((size_t)d);
         break;
      case 2: t.dtype = (int)f.v; break;
      case 4:
         if (f.wt == 2)
            for (size_t i = 0; i + 4 <= f.bytes.n; i += 4) {
               uint32_t b;
               std::memcpy(&b, f.bytes.p + i, 4);
               t.floats.push_back(AsFloat(b));
            }
         else
            t.floats.push_back(AsFloat((uint32_t)f.v));
         break;
      case 5:
      case 7:
         for (auto v : PackedInts(f))
            t.ints.push_back(v);
         break;
      case 8: t.name = Str(f); break;
      case 9: t.raw.assign(f.bytes.p, f.bytes.p + f.bytes.n); break;
      default: break;
      }
   }
   return t;
}

struct Attr {
   std::string s;
   int64_t i = 0;
   float f = 0;
   std::vector<int64_t> ints;
   std::vector<float> floats;
   Slice tensor; // a TensorProto (the `value` of a Constant node), inside the file's buffer
   bool has_i = false, has_f = false, has_s = false;
};

struct Node {
   std::string op, name;
   std::vector<std::string> in, out;
   std::map<std::string, Attr> attrs;
};

Node ParseNode(Slice s)
{
   Node n;
   Reader r(s);
   Field f;
   while (r.Next(f)) {
      switch (f.no) {
      case 1: n.in.push_back(Str(f)); break;
      case 2: n.out.push_back(Str(f)); break;
      case 3: n.name = Str(f); break;
      case 4: n.op = Str(f); break;
      case 5: {
         Attr a;
         std::string an;
         Reader ra(f.bytes);
         Field g;
         while (ra.Next(g)) {
            switch (g.no) {
            case 1: an = Str(g); break;
            case 2: a.f = AsFloat((uint32_t)g.v); a.has_f = true; break;
            case 3: a.i = (int64_t)g.v; a.has_i = true; break;
            case 4: a.s = Str(g); a.has_s = true; break;
            case 5:
               if (g.wt != 2)
                  throw std::runtime_error("SOFIE ONNX parser: attribute tensor should be length-delimited");
               a.tensor = g.bytes;
               break;
            case 7: AppendFloats(g, a.floats); break;
            case 8:
               for (auto v : PackedInts(g))
                  a.ints.push_back(v);
               break;
            default: break;
            }
         }
         n.attrs[an] = a;
      } break;
      default: break;
      }
   }
   return n;
}

struct ValueInfo {
   std::string name;
   int elem_type = 1;
   std::vector<size_t> shape;
   std::vector<Dim> dims; // the same with named parameters kept
   bool symbolic = false;
};

ValueInfo ParseValueInfo(Slice s)
{
   ValueInfo v;
   Reader r(s);
   Field f;
   while (r.Next(f)) {
      if (f.no == 1)
         v.name = Str(f);
      else if (f.no == 2) {
         Reader rt(f.bytes);
         Field t;
         while (rt.Next(t))
            if (t.no == 1) { // tensor_type
               Reader rtt(t.bytes);
               Field u;
               while (rtt.Next(u)) {
                  if (u.no == 1)
                     v.elem_type = (int)u.v;
                  else if (u.no == 2) { // shape
                     Reader rs(u.bytes);
                     Field d;
                     while (rs.Next(d))
                        if (d.no == 1) {
                           Reader rd(d.bytes);
                           Field x;
                           bool value = false;
                           std::string param;
                           while (rd.Next(x))
                              if (x.no == 1) {
                                 v.shape.push_back((size_t)x.v);
                                 v.dims.push_back(Dim((size_t)x.v));
                                 value = true;
                              } else if (x.no == 2) {
                                 param = Str(x);
                              }
                           if (!value) {
                              v.shape.push_back(0);
                              v.dims.push_back(Dim(param.empty() ? std::string("batch") : param, 1));
                              v.symbolic = true;
                           }
                        }
                  }
               }
            }
      }
   }
   return v;
}

std::vector<size_t> ToSizes(const std::vector<int64_t> &v) { return std::vector<size_t>(v.begin(), v.end()); }

} // namespace

std::unique_ptr<RModel> RModelParser_ONNX::Parse(std::string filename, bool verbose, std::string modelName)
{
   std::ifstream in(filename, std::ios::binary);
   if (!in.is_open())
      throw std::runtime_error("SOFIE ONNX parser: failed to open " + filename);
   std::vector<uint8_t> buf((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
   Slice graph;
   {
      Reader r(Slice{buf.data(), buf.size()});
      Field f;
      while (r.Next(f))
         if (f.no == 7)
            graph = f.bytes;
   }
   if (!graph.p)
      throw std::runtime_error("SOFIE ONNX parser: " + filename + " holds no graph");
   std::vector<Node> nodes;
   std::vector<Tensor> inits;
   std::vector<ValueInfo> inputs, outputs;
   {
      Reader r(graph);
      Field f;
      while (r.Next(f)) {
         if (f.no == 1)
            nodes.push_back(ParseNode(f.bytes));
         else if (f.no == 5)
            inits.push_back(ParseTensor(f.bytes));
         else if (f.no == 11)
            inputs.push_back(ParseValueInfo(f.bytes));
         else if (f.no == 12)
            outputs.push_back(ParseValueInfo(f.bytes));
      }
   }
   // A Constant node is an initializer under its output's name (the reference registers it as one when parsing,
   // parsers/src/ParseConstant.cxx): exporters write the shapes, axes and indices of Reshape / Slice / Gather this way.
   for (auto it = nodes.begin(); it != nodes.end();) {
      if (it->op != "Constant") {
         ++it;
         continue;
      }
      if (it->out.size() != 1)
         throw std::runtime_error("SOFIE ONNX parser: Constant " + it->name + " must have one output");
      Tensor t;
      auto has = [&](const char *a) { return it->attrs.count(a) != 0; };
      if (has("value") && it->attrs["value"].tensor.p) {
         t = ParseTensor(it->attrs["value"].tensor);
      } else if (has("value_float")) {
         t.dtype = static_cast<int>(ETensorType::FLOAT);
         t.floats = {it->attrs["value_float"].f};
      } else if (has("value_int")) {
         t.dtype = static_cast<int>(ETensorType::INT64);
         t.ints = {it->attrs["value_int"].i};
      } else if (has("value_ints")) {
         t.dtype = static_cast<int>(ETensorType::INT64);
         t.ints = it->attrs["value_ints"].ints;
         t.dims = {t.ints.size()};
      } else if (has("value_floats")) {
         t.dtype = static_cast<int>(ETensorType::FLOAT);
         t.floats = it->attrs["value_floats"].floats;
         t.dims = {t.floats.size()};
      } else {
         throw std::runtime_error("SOFIE ONNX parser: Constant " + it->name + " has no value, value_float(s) or value_int(s) attribute");
      }
      t.name = it->out[0];
      inits.push_back(std::move(t));
      it = nodes.erase(it);
   }
   auto model = std::make_unique<RModel>(modelName.empty() ? filename : modelName);
   std::map<std::string, bool> isInit;
   for (auto &t : inits) {
      isInit[t.name] = true;
      const ETensorType ty = static_cast<ETensorType>(t.dtype);
      const size_t len = CheckedShapeLength(t.dims, t.name);
      const size_t esz = GetTypeSize(ty);
      if (esz == 0)
         throw std::runtime_error("SOFIE ONNX parser: initializer " + t.name + " has an unsupported data type " + std::to_string(t.dtype));
      // the payload decides how much is allocated, not the dimensions the file claims
      const size_t have = !t.raw.empty() ? t.raw.size() / esz : ty == ETensorType::FLOAT ? t.floats.size() : t.ints.size();
      if (have != len)
         throw std::runtime_error("SOFIE ONNX parser: initializer " + t.name + " holds " + std::to_string(have) + " values, its shape asks for " +
                                  std::to_string(len));
      std::vector<uint8_t> data(len * esz);
      if (!t.raw.empty()) {
         if (t.raw.size() != data.size())
            throw std::runtime_error("SOFIE ONNX parser: initializer " + t.name + " has raw data of the wrong size");
         data = t.raw;
      } else if (ty == ETensorType::FLOAT) {
         if (t.floats.size() != len)
            throw std::runtime_error("SOFIE ONNX parser: initializer " + t.name + " has the wrong number of values");
         std::memcpy(data.data(), t.floats.data(), data.size());
      } else {
         if (t.ints.size() != len)
            throw std::runtime_error("SOFIE ONNX parser: initializer " + t.name + " has the wrong number of values");
         for (size_t i = 0; i < len; ++i) {
            int64_t v = t.ints[i];
            std::memcpy(data.data() + i * esz, &v, esz); // little endian: the low bytes
         }
      }
      model->AddInitializedTensor(t.name, ty, t.dims, data.data());
   }
   for (auto &v : inputs) {
      if (isInit.count(v.name))
         continue;
      if (v.symbolic) // a named leading dimension: the batch, fixed at generation (batchSize) or by the Session
         model->AddInputTensorInfo(v.name, static_cast<ETensorType>(v.elem_type), v.dims);
      else
         model->AddInputTensorInfo(v.name, static_cast<ETensorType>(v.elem_type), v.shape);
      model->AddInputTensorName(v.name);
   }
   std::map<std::string, int> uses;
   for (auto &n : nodes)
      for (auto &i : n.in)
         uses[i]++;
   auto attrI = [](const Node &n, const char *k, int64_t def) { auto f = n.attrs.find(k); return f == n.attrs.end() || !f->second.has_i ? def : f->second.i; };
   auto attrF = [](const Node &n, const char *k, float def) { auto f = n.attrs.find(k); return f == n.attrs.end() || !f->second.has_f ? def : f->second.f; };
   auto attrS = [](const Node &n, const char *k, const char *def) { auto f = n.attrs.find(k); return f == n.attrs.end() || !f->second.has_s ? std::string(def) : f->second.s; };
   auto attrV = [](const Node &n, const char *k) { auto f = n.attrs.find(k); return f == n.attrs.end() ? std::vector<size_t>{} : ToSizes(f->second.ints); };

   std::vector<bool> consumed(nodes.size(), false);

   // ---- parse-time rewrites of the reference (parsers/src/RModelParser_ONNX.cxx:1116-1140, 1186-1207) ----
   // Element types as far as the rewrites need them: graph inputs and initializers are known, an operator's output
   // takes the type its definition gives it.
   std::map<std::string, int> typeOf;
   for (auto &t : inits)
      typeOf[t.name] = t.dtype;
   for (auto &v : inputs)
      if (!typeOf.count(v.name))
         typeOf[v.name] = v.elem_type;
   std::map<std::string, size_t> rankOf;
   for (auto &t : inits)
      rankOf[t.name] = t.dims.size();
   for (auto &v : inputs)
      if (!rankOf.count(v.name))
         rankOf[v.name] = v.shape.size();
   auto isGraphOutput = [&](const std::string &name) {
      for (auto &o : outputs)
         if (o.name == name)
            return true;
      return false;
   };
   auto singleReader = [&](const std::string &name) -> size_t {
      size_t found = nodes.size(), count = 0;
      for (size_t j = 0; j < nodes.size(); ++j)
         for (auto &in : nodes[j].in)
            if (in == name) {
               found = j;
               ++count;
            }
      return count == 1 ? found : nodes.size();
   };
   std::map<std::string, std::string> transposedFrom; // output of an absorbed Transpose -> its input
   for (size_t i = 0; i < nodes.size(); ++i) {
      Node &n = nodes[i];
      if (n.in.empty() || n.out.empty())
         continue;
      const int inType = typeOf.count(n.in[0]) ? typeOf[n.in[0]] : 0;
      // a Cast to the type its input already has changes nothing: its output becomes another name of the input
      if (n.op == "Cast" && n.in.size() == 1 && n.out.size() == 1 && !isGraphOutput(n.out[0]) && inType != 0 &&
          attrI(n, "to", -1) == inType) {
         for (size_t j = i + 1; j < nodes.size(); ++j)
            for (auto &in : nodes[j].in)
               if (in == n.out[0])
                  in = n.in[0];
         consumed[i] = true;
         continue;
      }
      // Transpose of the last two axes whose only reader is a MatMul: the product reads the operand transposed
      if (n.op == "Transpose" && n.in.size() == 1 && n.out.size() == 1 && !isGraphOutput(n.out[0]) && inType == 1) {
         const size_t reader = singleReader(n.out[0]);
         bool lastTwo = false;
         auto perm = n.attrs.find("perm");
         if (perm == n.attrs.end()) {
            lastTwo = rankOf.count(n.in[0]) && rankOf[n.in[0]] == 2; // the default reverses every axis: a matrix transpose at rank 2 only
         } else {
            const auto &p = perm->second.ints;
            lastTwo = p.size() >= 2;
            for (size_t a = 0; lastTwo && a + 2 < p.size(); ++a)
               lastTwo = p[a] == (int64_t)a;
            lastTwo = lastTwo && p[p.size() - 2] == (int64_t)p.size() - 1 && p[p.size() - 1] == (int64_t)p.size() - 2;
         }
         if (lastTwo && reader < nodes.size() && nodes[reader].op == "MatMul" && nodes[reader].in.size() == 2) {
            transposedFrom[n.out[0]] = n.in[0];
            consumed[i] = true;
            continue;
         }
      }
      // element type and rank of what this node produces
      int outType = inType;
      if (n.op == "QuantizeLinear" || n.op == "QLinearConv" || n.op == "QLinearMatMul" || n.op == "QGemm")
         outType = 3;
      else if (n.op == "MatMulInteger" || n.op == "ConvInteger")
         outType = 6;
      else if (n.op == "DequantizeLinear")
         outType = 1;
      else if (n.op == "Cast")
         outType = (int)attrI(n, "to", 0);
      typeOf[n.out[0]] = outType;
      if (rankOf.count(n.in[0]) && (n.op == "Relu" || n.op == "Cast" || n.op == "Transpose" || n.op == "Identity"))
         rankOf[n.out[0]] = rankOf[n.in[0]];
   }
   uses.clear(); // the aliases and absorbed nodes changed who reads what
   for (size_t j = 0; j < nodes.size(); ++j)
      if (!consumed[j])
         for (auto &in : nodes[j].in)
            uses[in]++;

   for (size_t i = 0; i < nodes.size(); ++i) {
      if (consumed[i])
         continue;
      const Node &n = nodes[i];
      if (verbose)
         std::cout << "SOFIE HIP parser: " << n.op << " " << n.name << "\n";
      {
         // a node must name the inputs its operator reads below and one output, whatever the file claims
         static const std::map<std::string, size_t> minInputs = {
            {"Gemm", 2}, {"MatMul", 2}, {"Add", 2}, {"Sub", 2}, {"Mul", 2}, {"Div", 2}, {"Pow", 2}, {"Conv", 2}, {"QuantizeLinear", 2}, {"DequantizeLinear", 2}, {"BatchNormalization", 5},
            {"MatMulInteger", 2}, {"ConvInteger", 2}, {"QLinearConv", 8}, {"QLinearMatMul", 8}, {"QGemm", 9}};
         auto f = minInputs.find(n.op);
         const size_t need = f == minInputs.end() ? 1 : f->second;
         if (n.in.size() < need || n.out.empty())
            throw std::runtime_error("SOFIE ONNX parser: node " + n.op + (n.name.empty() ? "" : " (" + n.name + ")") + " has " +
                                     std::to_string(n.in.size()) + " inputs and " + std::to_string(n.out.size()) + " outputs; at least " +
                                     std::to_string(need) + " and 1 are needed");
      }
      if (n.op == "Gemm") {
         if (n.in.size() > 2 && !n.in[2].empty())
            model->AddOperator(std::make_unique<ROperator_Gemm<float>>(attrF(n, "alpha", 1.f), attrF(n, "beta", 1.f), attrI(n, "transA", 0),
                                                                       attrI(n, "transB", 0), n.in[0], n.in[1], n.in[2], n.out[0]));
         else
            model->AddOperator(std::make_unique<ROperator_Gemm<float>>(attrF(n, "alpha", 1.f), attrF(n, "beta", 1.f), attrI(n, "transA", 0),
                                                                       attrI(n, "transB", 0), n.in[0], n.in[1], n.out[0]));
      } else if (n.op == "MatMul") {
         // MatMul whose only consumer is an Add of an initializer: one Gemm with bias
         size_t addIdx = nodes.size();
         if (uses[n.out[0]] == 1)
            for (size_t j = i + 1; j < nodes.size(); ++j)
               if (nodes[j].op == "Add" && nodes[j].in.size() == 2 && (nodes[j].in[0] == n.out[0] || nodes[j].in[1] == n.out[0])) {
                  const std::string &other = nodes[j].in[0] == n.out[0] ? nodes[j].in[1] : nodes[j].in[0];
                  if (isInit.count(other))
                     addIdx = j;
                  break;
               }
         // operands that an absorbed Transpose produced are read transposed from its input
         const bool tA = transposedFrom.count(n.in[0]) != 0, tB = transposedFrom.count(n.in[1]) != 0;
         const std::string opA = tA ? transposedFrom[n.in[0]] : n.in[0], opB = tB ? transposedFrom[n.in[1]] : n.in[1];
         if (addIdx < nodes.size()) {
            const Node &a = nodes[addIdx];
            const std::string &bias = a.in[0] == n.out[0] ? a.in[1] : a.in[0];
            model->AddOperator(std::make_unique<ROperator_Gemm<float>>(1.f, 1.f, tA ? 1 : 0, tB ? 1 : 0, opA, opB, bias, a.out[0]));
            consumed[addIdx] = true;
         } else {
            model->AddOperator(std::make_unique<ROperator_Gemm<float>>(1.f, 0.f, tA ? 1 : 0, tB ? 1 : 0, opA, opB, n.out[0]));
         }
      } else if (n.op == "Relu") {
         model->AddOperator(std::make_unique<ROperator_Relu<float>>(n.in[0], n.out[0]));
      } else if (n.op == "Sigmoid") {
         model->AddOperator(std::make_unique<ROperator_Sigmoid<float>>(n.in[0], n.out[0]));
      } else if (n.op == "Tanh") {
         model->AddOperator(std::make_unique<ROperator_Tanh<float>>(n.in[0], n.out[0]));
      } else if (n.op == "LeakyRelu") {
         model->AddOperator(std::make_unique<ROperator_LeakyRelu<float>>(attrF(n, "alpha", 0.01f), n.in[0], n.out[0]));
      } else if (n.op == "Gelu") {
         model->AddOperator(std::make_unique<ROperator_Gelu<float>>(attrS(n, "approximate", "none"), n.in[0], n.out[0]));
      } else if (n.op == "Reciprocal" || n.op == "Sqrt" || n.op == "Neg" || n.op == "Exp" || n.op == "Log" || n.op == "Sin" || n.op == "Cos" ||
                 n.op == "Abs" || n.op == "Softplus" || n.op == "Atan" || n.op == "Floor" || n.op == "Asinh" || n.op == "Acosh" || n.op == "Atanh") {
         // the reference's ROperator_BasicUnary family (parsers/src/ParseBasicUnary.cxx)
         static const std::map<std::string, EActivationType> kinds = {
            {"Reciprocal", EActivationType::RECIPROCAL}, {"Sqrt", EActivationType::SQRT}, {"Neg", EActivationType::NEG}, {"Exp", EActivationType::EXP},
            {"Log", EActivationType::LOG}, {"Sin", EActivationType::SIN}, {"Cos", EActivationType::COS}, {"Abs", EActivationType::ABS},
            {"Softplus", EActivationType::SOFTPLUS}, {"Atan", EActivationType::ATAN}, {"Floor", EActivationType::FLOOR},
            {"Asinh", EActivationType::ASINH}, {"Acosh", EActivationType::ACOSH}, {"Atanh", EActivationType::ATANH}};
         model->AddOperator(std::make_unique<ROperator_Activation>(kinds.at(n.op), 0.f, n.in[0], n.out[0]));
      } else if (n.op == "Selu") {
         model->AddOperator(std::make_unique<ROperator_Selu<float>>(attrF(n, "alpha", 1.67326319217681884765625f),
                                                                    attrF(n, "gamma", 1.05070102214813232421875f), n.in[0], n.out[0]));
      } else if (n.op == "Elu") {
         model->AddOperator(std::make_unique<ROperator_Elu<float>>(attrF(n, "alpha", 1.0f), n.in[0], n.out[0]));
      } else if (n.op == "Erf") {
         model->AddOperator(std::make_unique<ROperator_Erf<float>>(n.in[0], n.out[0]));
      } else if (n.op == "HardSigmoid") {      // parsers/src/ParseHardSigmoid.cxx:20-33
         model->AddOperator(std::make_unique<ROperator_HardSigmoid<float>>(attrF(n, "alpha", 0.2f), attrF(n, "beta", 0.5f), n.in[0], n.out[0]));
      } else if (n.op == "HardSwish") {
         model->AddOperator(std::make_unique<ROperator_HardSwish<float>>(n.in[0], n.out[0]));
      } else if (n.op == "Swish") {
         model->AddOperator(std::make_unique<ROperator_Swish<float>>(n.in[0], n.out[0]));
      } else if (n.op == "Identity") {
         model->AddOperator(std::make_unique<ROperator_Identity<float>>(n.in[0], n.out[0]));
      } else if (n.op == "Clip") {
         // bounds: attributes up to opset 10, optional scalar initializers (inputs 1 and 2) from opset 11 on; absent = unbounded
         float lo = attrF(n, "min", std::numeric_limits<float>::lowest()), hi = attrF(n, "max", std::numeric_limits<float>::max());
         if (n.in.size() > 1 && !n.in[1].empty())
            lo = model->GetScalarInitializer(n.in[1]);
         if (n.in.size() > 2 && !n.in[2].empty())
            hi = model->GetScalarInitializer(n.in[2]);
         model->AddOperator(std::make_unique<ROperator_Clip<float>>(n.in[0], n.out[0], lo, hi));
      } else if (n.op == "Add") {
         model->AddOperator(std::make_unique<ROperator_BasicBinary<float, Add>>(n.in[0], n.in[1], n.out[0]));
      } else if (n.op == "Sub") {
         model->AddOperator(std::make_unique<ROperator_BasicBinary<float, Sub>>(n.in[0], n.in[1], n.out[0]));
      } else if (n.op == "Mul") {
         model->AddOperator(std::make_unique<ROperator_BasicBinary<float, Mul>>(n.in[0], n.in[1], n.out[0]));
      } else if (n.op == "Div") {
         model->AddOperator(std::make_unique<ROperator_BasicBinary<float, Div>>(n.in[0], n.in[1], n.out[0]));
      } else if (n.op == "Pow") {
         model->AddOperator(std::make_unique<ROperator_BasicBinary<float, Pow>>(n.in[0], n.in[1], n.out[0]));
      } else if (n.op == "Max" || n.op == "Min" || n.op == "Sum" || n.op == "Mean") {
         // the reference's ROperator_BasicNary (parsers/src/ParseBasicNary.cxx) as a left fold of pairwise steps: std::max({a, b, c})
         // is max(max(a, b), c), a + b + c is (a + b) + c, and Mean's last step also divides by the number of operands
         const size_t count = n.in.size();
         if (count == 1) {
            model->AddOperator(std::make_unique<ROperator_Identity<float>>(n.in[0], n.out[0]));
         } else {
            std::string acc = n.in[0];
            for (size_t i = 1; i < count; ++i) {
               const bool last = i + 1 == count;
               const std::string out = last ? n.out[0] : n.out[0] + "_fold" + std::to_string(i);
               if (n.op == "Max")
                  model->AddOperator(std::make_unique<ROperator_BasicBinary<float, PairMax>>(acc, n.in[i], out));
               else if (n.op == "Min")
                  model->AddOperator(std::make_unique<ROperator_BasicBinary<float, PairMin>>(acc, n.in[i], out));
               else if (n.op == "Mean" && last)
                  model->AddOperator(std::make_unique<ROperator_BasicBinary<float, AddThenDivide>>(acc, n.in[i], out, static_cast<float>(count)));
               else
                  model->AddOperator(std::make_unique<ROperator_BasicBinary<float, Add>>(acc, n.in[i], out));
               acc = out;
            }
         }
      } else if (n.op == "Conv") {
         std::string bias = n.in.size() > 2 ? n.in[2] : "";
         std::string out = n.out[0];
         // Conv without a bias whose only reader adds a one-dimensional initializer: that initializer is taken as the
         // convolution's per-channel bias, as the reference's parser does (IsConvBiasAdd, RModelParser_ONNX.cxx:1065-1075, 1203-1207)
         if (n.in.size() <= 2 && uses[n.out[0]] == 1 && !isGraphOutput(n.out[0])) {
            const size_t j = singleReader(n.out[0]);
            if (j < nodes.size() && !consumed[j] && nodes[j].op == "Add" && nodes[j].in.size() == 2 && !nodes[j].out.empty()) {
               const std::string &other = nodes[j].in[0] == n.out[0] ? nodes[j].in[1] : nodes[j].in[0];
               if (isInit.count(other) && rankOf.count(other) && rankOf[other] == 1) {
                  bias = other;
                  out = nodes[j].out[0];
                  consumed[j] = true;
               }
            }
         }
         model->AddOperator(std::make_unique<ROperator_Conv<float>>(attrS(n, "auto_pad", "NOTSET"), attrV(n, "dilations"), (size_t)attrI(n, "group", 1),
                                                                    attrV(n, "kernel_shape"), attrV(n, "pads"), attrV(n, "strides"), n.in[0],
                                                                    n.in[1], bias, out));
      } else if (n.op == "GlobalAveragePool") {
         model->AddOperator(std::make_unique<ROperator_Pool<float>>(GlobalAveragePool, n.in[0], n.out[0]));
      } else if (n.op == "LayerNormalization") {
         if (n.in.size() < 2)
            throw std::runtime_error("SOFIE ONNX parser: LayerNormalization " + n.name + " needs X and Scale");
         model->AddOperator(std::make_unique<ROperator_LayerNormalization<float>>(
            (int)attrI(n, "axis", -1), attrF(n, "epsilon", 1e-5f), (size_t)attrI(n, "stash_type", 1), n.in[0], n.in[1], n.in.size() > 2 ? n.in[2] : "", n.out[0],
            n.out.size() > 1 ? n.out[1] : "", n.out.size() > 2 ? n.out[2] : ""));
      } else if (n.op.rfind("Reduce", 0) == 0) {
         // keepdims = 1 and the axes attribute (before opset 13 / 18) or the axes input (parsers/src/ParseReduce.cxx:41-62)
         auto f = n.attrs.find("axes");
         const std::vector<int64_t> axes = f == n.attrs.end() ? std::vector<int64_t>{} : f->second.ints;
         const int keepdims = (int)attrI(n, "keepdims", 1);
         const std::string axesName = n.in.size() > 1 ? n.in[1] : "";
         if (n.op == "ReduceMean")
            model->AddOperator(std::make_unique<ROperator_Reduce<ReduceMean>>(keepdims, axes, n.in[0], axesName, n.out[0]));
         else if (n.op == "ReduceSum")
            model->AddOperator(std::make_unique<ROperator_Reduce<ReduceSum>>(keepdims, axes, n.in[0], axesName, n.out[0]));
         else if (n.op == "ReduceSumSquare")
            model->AddOperator(std::make_unique<ROperator_Reduce<ReduceSumSquare>>(keepdims, axes, n.in[0], axesName, n.out[0]));
         else if (n.op == "ReduceProd")
            model->AddOperator(std::make_unique<ROperator_Reduce<ReduceProd>>(keepdims, axes, n.in[0], axesName, n.out[0]));
         else if (n.op == "ReduceL2")
            model->AddOperator(std::make_unique<ROperator_Reduce<ReduceL2>>(keepdims, axes, n.in[0], axesName, n.out[0]));
         else if (n.op == "ReduceMax")
            model->AddOperator(std::make_unique<ROperator_Reduce<ReduceMax>>(keepdims, axes, n.in[0], axesName, n.out[0]));
         else if (n.op == "ReduceMin")
            model->AddOperator(std::make_unique<ROperator_Reduce<ReduceMin>>(keepdims, axes, n.in[0], axesName, n.out[0]));
         else
            throw std::runtime_error("SOFIE - Reduce op mode not supported.");
      } else if (n.op == "Softmax" || n.op == "LogSoftmax") {
         model->AddOperator(std::make_unique<ROperator_Softmax>(attrI(n, "axis", -1), n.in[0], n.out[0], n.op == "LogSoftmax"));
      } else if (n.op == "MaxPool" || n.op == "AveragePool") {
         // attributes as parsers/src/ParsePool.cxx:37-63 reads them: count_include_pad belongs to AveragePool,
         // storage_order and dilations to MaxPool
         const bool isMax = n.op == "MaxPool";
         if (n.out.size() > 1 && !n.out[1].empty())
            throw std::runtime_error("SOFIE ONNX parser: MaxPool " + n.name + " asks for the Indices output, which is not supported");
         RAttributes_Pool attr;
         attr.auto_pad = attrS(n, "auto_pad", "NOTSET");
         attr.ceil_mode = (int)attrI(n, "ceil_mode", 0);
         attr.count_include_pad = isMax ? 0 : (int)attrI(n, "count_include_pad", 0);
         attr.storage_order = isMax ? (int)attrI(n, "storage_order", 0) : 0;
         if (isMax)
            attr.dilations = attrV(n, "dilations");
         attr.kernel_shape = attrV(n, "kernel_shape");
         attr.pads = attrV(n, "pads");
         attr.strides = attrV(n, "strides");
         model->AddOperator(std::make_unique<ROperator_Pool<float>>(isMax ? MaxPool : AveragePool, attr, n.in[0], n.out[0]));
      } else if (n.op == "QuantizeLinear") {
         model->AddOperator(std::make_unique<ROperator_QuantizeLinear>(n.in[0], n.in[1], n.out[0]));
      } else if (n.op == "DequantizeLinear") {
         model->AddOperator(std::make_unique<ROperator_DequantizeLinear>(n.in[0], n.in[1], n.out[0]));
      } else if (n.op == "BatchNormalization") {
         if (n.in.size() != 5)
            throw std::runtime_error("SOFIE ONNX parser: BatchNormalization " + n.name + " needs 5 inputs");
         model->AddOperator(std::make_unique<ROperator_BatchNormalization<float>>(attrF(n, "epsilon", 1e-5f), attrF(n, "momentum", 0.9f),
                                                                                   (size_t)attrI(n, "training_mode", 0), n.in[0], n.in[1], n.in[2],
                                                                                   n.in[3], n.in[4], n.out[0]));
      } else if (n.op == "QLinearConv") {
         if (n.in.size() < 8)
            throw std::runtime_error("SOFIE ONNX parser: QLinearConv " + n.name + " needs 8 or 9 inputs");
         model->AddOperator(std::make_unique<ROperator_QConv>(attrS(n, "auto_pad", "NOTSET"), attrV(n, "dilations"), (size_t)attrI(n, "group", 1),
                                                              attrV(n, "kernel_shape"), attrV(n, "pads"), attrV(n, "strides"), n.in[0], n.in[1],
                                                              n.in[2], n.in[3], n.in[4], n.in[5], n.in[6], n.in[7],
                                                              n.in.size() > 8 ? n.in[8] : "", n.out[0]));
      } else if (n.op == "ConvInteger") {
         model->AddOperator(ROperator_QConv::MakeConvInteger(attrS(n, "auto_pad", "NOTSET"), attrV(n, "dilations"), (size_t)attrI(n, "group", 1),
                                                             attrV(n, "kernel_shape"), attrV(n, "pads"), attrV(n, "strides"), n.in[0], n.in[1],
                                                             n.in.size() > 2 ? n.in[2] : "", n.in.size() > 3 ? n.in[3] : "", n.out[0]));
      } else if (n.op == "QLinearMatMul") {
         // y = sat8(rne(acc * ((a_scale * b_scale[n]) / y_scale))): the multipliers are formed here, once, in fp32
         if (n.in.size() != 8)
            throw std::runtime_error("SOFIE ONNX parser: QLinearMatMul " + n.name + " needs 8 inputs");
         for (int z : {2, 5, 7}) {
            const std::string zn = UTILITY::Clean_name(n.in[z]);
            if (!model->IsInitializedTensor(zn) || model->GetTensorType(zn) != ETensorType::INT8)
               throw std::runtime_error("SOFIE ONNX parser: QLinearMatMul zero point " + n.in[z] + " must be an int8 initializer");
            const auto *p = static_cast<const int8_t *>(model->GetInitializedTensorData(zn).get());
            for (size_t k = 0; k < ConvertShapeToLength(model->GetTensorShape(zn)); ++k)
               if (p[k] != 0)
                  throw std::runtime_error("SOFIE ONNX parser: QLinearMatMul zero point " + n.in[z] + " is not 0; symmetric quantisation only");
         }
         const float as = model->GetScalarInitializer(n.in[1]), ys = model->GetScalarInitializer(n.in[6]);
         const std::string bsn = UTILITY::Clean_name(n.in[4]), bn = UTILITY::Clean_name(n.in[3]);
         if (!model->IsInitializedTensor(bsn) || model->GetTensorType(bsn) != ETensorType::FLOAT || !model->IsInitializedTensor(bn))
            throw std::runtime_error("SOFIE ONNX parser: QLinearMatMul needs an initializer B with a float scale initializer");
         const size_t ncols = model->GetTensorShape(bn).back(), nbs = ConvertShapeToLength(model->GetTensorShape(bsn));
         if (nbs != 1 && nbs != ncols)
            throw std::runtime_error("SOFIE ONNX parser: QLinearMatMul scale of B must have 1 or N elements");
         const float *bs = static_cast<const float *>(model->GetInitializedTensorData(bsn).get());
         std::vector<float> mult(ncols);
         for (size_t c = 0; c < ncols; ++c) {
            volatile float prod = as * bs[nbs == 1 ? 0 : c];
            mult[c] = prod / ys;
         }
         const std::string mname = n.out[0] + "_requant_scale";
         model->AddInitializedTensor(mname, ETensorType::FLOAT, {ncols}, mult.data());
         auto op = std::make_unique<ROperator_QGemm>(n.in[0], n.in[3], n.out[0]);
         op->SetRequantize(mname, false);
         model->AddOperator(std::move(op));
      } else if (n.op == "QGemm") {
         // The contrib operator (domain com.microsoft): Y = sat8(rne((A x B + C) * ((a_scale * b_scale[n]) / y_scale))) with an
         // int32 bias C [N] that counts in units of a_scale * b_scale, i.e. is added to the accumulator.  Inputs: A, a_scale,
         // a_zero_point, B, b_scale, b_zero_point, C, y_scale, y_zero_point.  Symmetric quantisation, alpha = 1, a constant B
         // stored [K,N].
         if (n.in.size() != 9)
            throw std::runtime_error("SOFIE ONNX parser: QGemm " + n.name + " needs 9 inputs (the quantised output form)");
         if (attrF(n, "alpha", 1.f) != 1.f || attrI(n, "transA", 0) != 0 || attrI(n, "transB", 0) != 0)
            throw std::runtime_error("SOFIE ONNX parser: QGemm " + n.name + ": alpha = 1, transA = 0 and transB = 0 only");
         for (int z : {2, 5, 8}) {
            const std::string zn = UTILITY::Clean_name(n.in[z]);
            if (!model->IsInitializedTensor(zn) || model->GetTensorType(zn) != ETensorType::INT8)
               throw std::runtime_error("SOFIE ONNX parser: QGemm zero point " + n.in[z] + " must be an int8 initializer");
            const auto *p = static_cast<const int8_t *>(model->GetInitializedTensorData(zn).get());
            for (size_t k = 0; k < ConvertShapeToLength(model->GetTensorShape(zn)); ++k)
               if (p[k] != 0)
                  throw std::runtime_error("SOFIE ONNX parser: QGemm zero point " + n.in[z] + " is not 0; symmetric quantisation only");
         }
         const float as = model->GetScalarInitializer(n.in[1]), ys = model->GetScalarInitializer(n.in[7]);
         const std::string bsn = UTILITY::Clean_name(n.in[4]), bn = UTILITY::Clean_name(n.in[3]);
         if (!model->IsInitializedTensor(bsn) || model->GetTensorType(bsn) != ETensorType::FLOAT || !model->IsInitializedTensor(bn))
            throw std::runtime_error("SOFIE ONNX parser: QGemm needs an initializer B with a float scale initializer");
         const size_t ncols = model->GetTensorShape(bn).back(), nbs = ConvertShapeToLength(model->GetTensorShape(bsn));
         if (nbs != 1 && nbs != ncols)
            throw std::runtime_error("SOFIE ONNX parser: QGemm scale of B must have 1 or N elements");
         const float *bs = static_cast<const float *>(model->GetInitializedTensorData(bsn).get());
         std::vector<float> mult(ncols);
         for (size_t c = 0; c < ncols; ++c) {
            volatile float prod = as * bs[nbs == 1 ? 0 : c];
            mult[c] = prod / ys;
         }
         const std::string mname = n.out[0] + "_requant_scale";
         model->AddInitializedTensor(mname, ETensorType::FLOAT, {ncols}, mult.data());
         auto op = std::make_unique<ROperator_QGemm>(n.in[0], n.in[3], n.out[0]);
         if (!n.in[6].empty())
            op->SetBias(n.in[6]);
         op->SetRequantize(mname, false);
         model->AddOperator(std::move(op));
      } else if (n.op == "Flatten") {
         model->AddOperator(std::make_unique<ROperator_Reshape>(Flatten, (int)attrI(n, "axis", 1), n.in[0], "", n.out[0]));
      } else if (n.op == "Reshape") {
         if (n.in.size() < 2)
            throw std::runtime_error("SOFIE ONNX parser: Reshape " + n.name + " needs the shape as its second input");
         model->AddOperator(std::make_unique<ROperator_Reshape>(Reshape, (int)attrI(n, "allowzero", 0), n.in[0], n.in[1], n.out[0]));
      } else if (n.op == "Squeeze" || n.op == "Unsqueeze") {
         // the axes are an input from opset 13 on, an attribute before (parsers/src/ParseReshape.cxx:19-51)
         const ReshapeOpMode mode = n.op == "Squeeze" ? Squeeze : Unsqueeze;
         if (n.in.size() > 1 && !n.in[1].empty()) {
            model->AddOperator(std::make_unique<ROperator_Reshape>(mode, 0, n.in[0], n.in[1], n.out[0]));
         } else {
            auto f = n.attrs.find("axes");
            model->AddOperator(std::make_unique<ROperator_Reshape>(mode, f == n.attrs.end() ? std::vector<int64_t>{} : f->second.ints, n.in[0], n.out[0]));
         }
      } else if (n.op == "Slice") {
         // starts / ends / axes / steps are inputs from opset 10 on, attributes before (parsers/src/ParseSlice.cxx:19-47)
         if (n.in.size() > 1) {
            model->AddOperator(std::make_unique<ROperator_Slice<float, int64_t>>(n.in[0], std::vector<std::string>(n.in.begin() + 1, n.in.end()), n.out[0]));
         } else {
            auto ints = [&](const char *name) {
               auto f = n.attrs.find(name);
               return f == n.attrs.end() ? std::vector<int64_t>{} : f->second.ints;
            };
            model->AddOperator(std::make_unique<ROperator_Slice<float, int64_t>>(n.in[0], ints("starts"), ints("ends"), ints("axes"), n.out[0]));
         }
      } else if (n.op == "Split") {
         for (auto &kv : n.attrs)
            if (kv.first != "axis" && kv.first != "num_outputs")
               throw std::runtime_error("SOFIE ONNX Parser Split operator: attribute" + kv.first + "is not yet supported");
         model->AddOperator(std::make_unique<ROperator_Split>(n.in[0], n.in.size() > 1 ? n.in[1] : "", (int)attrI(n, "axis", 0), n.out));
      } else if (n.op == "Expand" || n.op == "Tile") {
         if (n.in.size() < 2)
            throw std::runtime_error("SOFIE ONNX parser: " + n.op + " " + n.name + " needs its second input");
         if (n.op == "Expand")
            model->AddOperator(std::make_unique<ROperator_Expand<float>>(n.in[0], n.in[1], n.out[0]));
         else
            model->AddOperator(std::make_unique<ROperator_Tile<float>>(n.in[1], n.in[0], n.out[0]));
      } else if (n.op == "Gather") {
         if (n.in.size() < 2)
            throw std::runtime_error("SOFIE ONNX parser: Gather " + n.name + " needs its indices");
         model->AddOperator(std::make_unique<ROperator_Gather>(attrI(n, "axis", 0), n.in[0], n.in[1], n.out[0]));
      } else if (n.op == "Transpose") {
         auto f = n.attrs.find("perm");
         model->AddOperator(std::make_unique<ROperator_Transpose<float>>(f == n.attrs.end() ? std::vector<int64_t>{} : f->second.ints, n.in[0], n.out[0]));
      } else if (n.op == "Concat") {
         model->AddOperator(std::make_unique<ROperator_Concat>(n.in, (int)attrI(n, "axis", 0), 0, n.out[0]));
      } else if (n.op == "MatMulInteger") {
         model->AddOperator(MakeMatMulInteger(n.in[0], n.in[1], n.out[0]));
      } else {
         throw std::runtime_error("SOFIE Operator type " + n.op + " is not yet supported");
      }
   }
   std::vector<std::string> outs;
   for (auto &o : outputs)
      outs.push_back(o.name);
   model->AddOutputTensorNameList(outs);
   return model;
}

} // namespace SOFIE_HIP
