// Test harness for Sessions emitted with Options::kStridedInput: the Gemm scenarios of the reference's
// tests/alpaka/TestAlpakaStridedInput.cxx (GemmBiasReluLayouts, GemmTransposedOperands, GemmWithoutUnitStrideThrows,
// InvalidStridesAreRejected, GemmBothOperandsStrided, GemmTransposedOperandsBothStrided, GemmOperandWithoutUnitStrideThrows,
// DynamicShapeStridedSubBatch) on the models of its tests/models/StridedInputModelGenerator.cxx, driven from Python through one C
// function.  Every layout runs three ways: host pointers, views of device memory on a 256-byte boundary (read in place) and
// views off it (copied into the Session's region first).  The expected values are the plain loops over the logical tensors.
// The device memory of the views is the arena of a second runtime context, so this file needs no HIP header.
#include "StridedGemmAB_GPU_HIP.hxx"
#include "StridedGemmABt_GPU_HIP.hxx"
#include "StridedGemmAllOptions_GPU_HIP.hxx"
#include "StridedGemmBiasRelu_GPU_HIP.hxx"
#include "StridedGemmDynamic_GPU_HIP.hxx"
#include "StridedGemmTransAB_GPU_HIP.hxx"

#include <cmath>
#include <cstring>
#include <functional>
#include <sstream>

namespace {
using Strides = std::vector<std::size_t>;

// A logical row-major tensor laid out in memory through strides; what lies between its elements holds 99.
struct Laid {
   std::vector<float> storage, logical;
   Laid(const std::vector<std::size_t> &shape, const Strides &strides, std::function<float(std::size_t)> value)
   {
      std::size_t length = 1, last = 0;
      for (std::size_t d = 0; d < shape.size(); ++d) {
         length *= shape[d];
         last += (shape[d] - 1) * strides[d];
      }
      storage.assign(last + 1, 99.f);
      logical.resize(length);
      for (std::size_t k = 0; k < length; ++k) {
         std::size_t rest = k, at = 0;
         for (std::size_t d = shape.size(); d-- > 0;) {
            at += (rest % shape[d]) * strides[d];
            rest /= shape[d];
         }
         logical[k] = value(k);
         storage[at] = logical[k];
      }
   }
};
float ramp(std::size_t k) { return 0.37f * float(k) - 2.f; }
float saw(std::size_t k) { return 0.1f * float(k % 7) - 0.3f; }

// the weights of the models (tools/emit_example_api.cxx): v[i] = scale * ((7 i) mod 11) - 0.5
std::vector<float> Weights(std::size_t n, float scale)
{
   std::vector<float> v(n);
   for (std::size_t i = 0; i < n; ++i)
      v[i] = scale * float((i * 7) % 11) - 0.5f;
   return v;
}
// Y[rows,4] = (relu)(X[rows,5] * W[5,4] + B)
std::vector<float> BiasProduct(const std::vector<float> &x, std::size_t rows, bool relu)
{
   const auto W = Weights(20, 0.1f), B = Weights(4, 0.3f);
   std::vector<float> y(rows * 4);
   for (std::size_t i = 0; i < rows; ++i)
      for (std::size_t j = 0; j < 4; ++j) {
         float acc = B[j];
         for (std::size_t k = 0; k < 5; ++k)
            acc += x[i * 5 + k] * W[k * 4 + j];
         y[i * 4 + j] = relu ? std::max(acc, 0.f) : acc;
      }
   return y;
}
bool Close(const std::vector<float> &got, const std::vector<float> &want)
{
   if (got.size() != want.size())
      return false;
   for (std::size_t i = 0; i < got.size(); ++i)
      if (!(std::fabs(got[i] - want[i]) <= 1e-5f * std::max(1.f, std::fabs(want[i]))))
         return false;
   return true;
}

// device memory for the views: consecutive 256-byte aligned pieces of the helper context's arena
struct DeviceArea {
   sofie_hip_ctx *ctx;
   std::size_t used = 0;
   float *put(const std::vector<float> &host, std::size_t misalign)
   {
      float *p = reinterpret_cast<float *>(static_cast<char *>(sofie_hip_arena_ptr(ctx, used))) + misalign;
      if (sofie_hip_upload(ctx, p, host.data(), host.size() * sizeof(float)) || sofie_hip_sync(ctx))
         throw std::runtime_error(sofie_hip_last_error());
      used += ((host.size() + misalign) * sizeof(float) + 511) / 256 * 256;
      return p;
   }
};

// runs a Session of one or two inputs three ways and compares each result with `want`
template <class SessionT, class View, class OutView>
bool ThreeWays(SessionT &s, const std::vector<const Laid *> &in, const std::vector<float> &want, sofie_hip_ctx *helper, std::string &why)
{
   std::vector<float> y;
   if constexpr (requires { s.infer(in[0]->storage.data()); }) {
      y = s.infer(in[0]->storage.data());
   } else {
      y = s.infer(in[0]->storage.data(), in[1]->storage.data());
   }
   if (!Close(y, want)) {
      why = "host pointers";
      return false;
   }
   for (std::size_t misalign : {std::size_t(0), std::size_t(3)}) {
      DeviceArea area{helper};
      std::vector<View> views;
      for (auto *l : in)
         views.push_back(View{area.put(l->storage, misalign), l->storage.size()});
      std::vector<float> zeros(want.size(), 0.f), got(want.size());
      float *out = area.put(zeros, misalign);
      std::vector<OutView> outs{OutView{out, want.size()}};
      s.infer(std::span<View const>(views), std::span<OutView>(outs));
      if (sofie_hip_download(helper, got.data(), out, got.size() * sizeof(float)) || sofie_hip_sync(helper))
         throw std::runtime_error(sofie_hip_last_error());
      if (!Close(got, want)) {
         why = misalign ? "views off the boundary" : "views in place";
         return false;
      }
   }
   return true;
}
} // namespace

extern "C" int run_strided_input(const char *dir, char *report, int len)
{
   std::ostringstream out;
   int failures = 0;
   auto expect = [&](bool ok, const std::string &what) {
      out << (ok ? "ok " : "FAIL ") << what << "\n";
      failures += ok ? 0 : 1;
   };
   auto name = [](const Strides &s) { return "{" + std::to_string(s[0]) + ", " + std::to_string(s[1]) + "}"; };
   sofie_hip_ctx *helper = nullptr;
   try {
      if (sofie_hip_ctx_create(&helper, 0, nullptr) || sofie_hip_arena_create(helper, 1 << 20, 256))
         throw std::runtime_error(sofie_hip_last_error());
      const std::string wBias = std::string(dir) + "/StridedGemmBiasRelu_GPU_HIP.dat", wTrans = std::string(dir) + "/StridedGemmTransAB_GPU_HIP.dat",
                        wDyn = std::string(dir) + "/StridedGemmDynamic_GPU_HIP.dat";
      std::string why;
      {
         // GemmBiasReluLayouts: row-major, row padded and column-major 3 x 5 inputs; no strides at all = contiguous
         using namespace SOFIE_StridedGemmBiasRelu;
         for (const Strides &st : {Strides{5, 1}, Strides{8, 1}, Strides{1, 3}, Strides{1, 6}}) {
            Laid x({3, 5}, st, ramp);
            Session s(wBias, {st});
            const bool ok = ThreeWays<Session, ViewConstF1D, ViewF1D>(s, {&x}, BiasProduct(x.logical, 3, true), helper, why);
            expect(ok, "Gemm + bias + Relu, input strides " + name(st) + (ok ? "" : ": " + why));
         }
         {
            Laid x({3, 5}, {5, 1}, ramp);
            Session s(wBias);
            expect(ThreeWays<Session, ViewConstF1D, ViewF1D>(s, {&x}, BiasProduct(x.logical, 3, true), helper, why), "no strides given: contiguous input");
            Session e(wBias, {Strides{}});
            expect(ThreeWays<Session, ViewConstF1D, ViewF1D>(e, {&x}, BiasProduct(x.logical, 3, true), helper, why), "an empty stride array: contiguous input");
         }
         // GemmWithoutUnitStrideThrows: the Session is built, the inference refuses
         {
            Laid x({3, 5}, {20, 2}, ramp);
            Session s(wBias, {{20, 2}});
            bool threw = false;
            try {
               s.infer(x.storage.data());
            } catch (const std::runtime_error &e) {
               threw = std::string(e.what()).find("without a unit stride") != std::string::npos;
            }
            expect(threw, "strides {20, 2} without a unit stride are refused by infer");
         }
         // InvalidStridesAreRejected: one array per input, one stride per dimension
         bool threw = false;
         try {
            Session s(wBias, {{5, 1}, {5, 1}});
         } catch (const std::runtime_error &e) {
            threw = std::string(e.what()).find("expected 1 input stride array(s)") != std::string::npos;
         }
         expect(threw, "two stride arrays for one input are rejected by the constructor");
         threw = false;
         try {
            Session s(wBias, {{5, 1, 1}});
         } catch (const std::runtime_error &e) {
            threw = std::string(e.what()).find("must have 2 element(s)") != std::string::npos;
         }
         expect(threw, "three strides for a 2-D input are rejected by the constructor");
         // a view that does not cover the padded rows is refused before anything runs
         {
            Laid x({3, 5}, {8, 1}, ramp);
            Session s(wBias, {{8, 1}});
            DeviceArea area{helper};
            std::vector<ViewConstF1D> in{ViewConstF1D{area.put(x.storage, 0), 15}};
            std::vector<float> zeros(12, 0.f);
            std::vector<ViewF1D> outs{ViewF1D{area.put(zeros, 0), 12}};
            threw = false;
            try {
               s.infer(std::span<ViewConstF1D const>(in), std::span<ViewF1D>(outs));
            } catch (const std::runtime_error &) {
               threw = true;
            }
            expect(threw, "a view of 15 elements for rows padded to 8 (21 elements) is refused");
         }
      }
      {
         // GemmTransposedOperands: Y = X^T * W^T with X stored 5 x 3
         using namespace SOFIE_StridedGemmTransAB;
         const auto W = Weights(20, 0.1f);
         for (const Strides &st : {Strides{3, 1}, Strides{8, 1}, Strides{1, 5}}) {
            Laid x({5, 3}, st, ramp);
            std::vector<float> want(12);
            for (std::size_t i = 0; i < 3; ++i)
               for (std::size_t j = 0; j < 4; ++j) {
                  float acc = 0;
                  for (std::size_t k = 0; k < 5; ++k)
                     acc += x.logical[k * 3 + i] * W[j * 5 + k];
                  want[i * 4 + j] = acc;
               }
            Session s(wTrans, {st});
            const bool ok = ThreeWays<Session, ViewConstF1D, ViewF1D>(s, {&x}, want, helper, why);
            expect(ok, "transposed operands, input strides " + name(st) + (ok ? "" : ": " + why));
         }
      }
      {
         // GemmBothOperandsStrided: Y = A[3,5] * B[5,4], both graph inputs
         using namespace SOFIE_StridedGemmAB;
         const std::vector<Strides> layoutsA{{5, 1}, {8, 1}, {1, 3}}, layoutsB{{4, 1}, {6, 1}, {1, 5}};
         for (std::size_t l = 0; l < layoutsA.size(); ++l) {
            Laid a({3, 5}, layoutsA[l], ramp), b({5, 4}, layoutsB[l], saw);
            std::vector<float> want(12, 0.f);
            for (std::size_t r = 0; r < 3; ++r)
               for (std::size_t c = 0; c < 4; ++c)
                  for (std::size_t k = 0; k < 5; ++k)
                     want[r * 4 + c] += a.logical[r * 5 + k] * b.logical[k * 4 + c];
            Session s("", {layoutsA[l], layoutsB[l]});
            const bool ok = ThreeWays<Session, ViewConstF1D, ViewF1D>(s, {&a, &b}, want, helper, why);
            expect(ok, "both operands strided, " + name(layoutsA[l]) + " and " + name(layoutsB[l]) + (ok ? "" : ": " + why));
         }
         // only the second input strided: the first keeps its planned region
         {
            Laid a({3, 5}, {5, 1}, ramp), b({5, 4}, {1, 7}, saw);
            std::vector<float> want(12, 0.f);
            for (std::size_t r = 0; r < 3; ++r)
               for (std::size_t c = 0; c < 4; ++c)
                  for (std::size_t k = 0; k < 5; ++k)
                     want[r * 4 + c] += a.logical[r * 5 + k] * b.logical[k * 4 + c];
            Session s("", {Strides{}, Strides{1, 7}});
            expect(ThreeWays<Session, ViewConstF1D, ViewF1D>(s, {&a, &b}, want, helper, why), "only the second operand strided");
         }
         // GemmOperandWithoutUnitStrideThrows
         Laid a({3, 5}, {5, 1}, ramp), b({5, 4}, {8, 2}, saw);
         Session s("", {{5, 1}, {8, 2}});
         bool threw = false;
         try {
            s.infer(a.storage.data(), b.storage.data());
         } catch (const std::runtime_error &e) {
            threw = std::string(e.what()).find("input tensor B has strides {8, 2}") != std::string::npos;
         }
         expect(threw, "second operand with strides {8, 2} is refused by infer, naming the tensor");
      }
      {
         // GemmTransposedOperandsBothStrided: Y = A^T * B^T with A stored 5 x 3 and B stored 4 x 5
         using namespace SOFIE_StridedGemmABt;
         const std::vector<Strides> layoutsA{{3, 1}, {8, 1}, {1, 5}}, layoutsB{{5, 1}, {7, 1}, {1, 4}};
         for (std::size_t l = 0; l < layoutsA.size(); ++l) {
            Laid a({5, 3}, layoutsA[l], ramp), b({4, 5}, layoutsB[l], saw);
            std::vector<float> want(12, 0.f);
            for (std::size_t r = 0; r < 3; ++r)
               for (std::size_t c = 0; c < 4; ++c)
                  for (std::size_t k = 0; k < 5; ++k)
                     want[r * 4 + c] += a.logical[k * 3 + r] * b.logical[c * 5 + k];
            Session s("", {layoutsA[l], layoutsB[l]});
            const bool ok = ThreeWays<Session, ViewConstF1D, ViewF1D>(s, {&a, &b}, want, helper, why);
            expect(ok, "both operands transposed and strided, " + name(layoutsA[l]) + " and " + name(layoutsB[l]) + (ok ? "" : ": " + why));
         }
      }
      {
         // DynamicShapeStridedSubBatch: maximum batch 8, a batch of 6 rows read from a matrix with leading dimension 7; then the
         // same rows stored column by column with 9 elements to a column
         using namespace SOFIE_StridedGemmDynamic;
         for (const Strides &st : {Strides{7, 1}, Strides{1, 9}}) {
            Laid x({6, 5}, st, ramp);
            Session s(wDyn, 8, {st});
            bool ok = Close(s.infer(6, x.storage.data()), BiasProduct(x.logical, 6, false));
            for (std::size_t misalign : {std::size_t(0), std::size_t(3)}) {
               DeviceArea area{helper};
               std::vector<ViewConstF1D> in{ViewConstF1D{area.put(x.storage, misalign), x.storage.size()}};
               std::vector<float> zeros(24, 0.f), got(24);
               float *o = area.put(zeros, misalign);
               std::vector<ViewF1D> outs{ViewF1D{o, 24}};
               s.infer(std::span<ViewConstF1D const>(in), std::span<ViewF1D>(outs), 6);
               if (sofie_hip_download(helper, got.data(), o, got.size() * sizeof(float)) || sofie_hip_sync(helper))
                  throw std::runtime_error(sofie_hip_last_error());
               ok = ok && Close(got, BiasProduct(x.logical, 6, false));
            }
            expect(ok, "run-time batch: 6 of at most 8 rows, input strides " + name(st));
         }
         Laid x({8, 5}, {5, 1}, ramp);
         Session s(wDyn, 8);
         expect(Close(s.infer(8, x.storage.data()), BiasProduct(x.logical, 8, false)), "run-time batch without strides: the current shape, contiguous");
      }
      {
         // every Session option at once: the caller's block holds the planned arena AND the region of the strided input
         using namespace SOFIE_StridedGemmAllOptions;
         const std::string wAll = std::string(dir) + "/StridedGemmAllOptions_GPU_HIP.safetensors";
         char *memory = static_cast<char *>(sofie_hip_arena_ptr(helper, 512 * 1024));
         std::size_t asked = 0, assignedPastPlan = 0;
         int freed = 0;
         MemoryProvider provider;
         provider.alloc = [&](std::size_t bytes) -> void * {
            asked = bytes;
            return memory;
         };
         provider.assign = [&](std::size_t off) -> void * {
            assignedPastPlan += off >= Session::ArenaBytes(8) ? 1 : 0;
            return memory + off;
         };
         provider.dealloc = [&](void *) { ++freed; };
         {
            Laid x({6, 5}, {7, 1}, ramp);
            Session s(provider, wAll, 8, {{7, 1}}, sofie_hip_stream(helper));
            // the input's extent at the maximum batch: 7 rows of 7 + 5 elements = 54 floats, rounded up to 256 bytes
            expect(asked == Session::ArenaBytes(8) + 256 && assignedPastPlan == 1, "caller's memory: the block is the planned arena plus the strided input's region");
            expect(s.stream() == sofie_hip_stream(helper) && Close(s.infer(6, x.storage.data()), BiasProduct(x.logical, 6, false)),
                   "caller's memory and stream, safetensors weights, run-time batch, input strides {7, 1}");
         }
         expect(freed == 1, "caller's memory: block returned once");
         {
            Laid x({8, 5}, {5, 1}, ramp);
            asked = 0;
            Session s(provider, wAll, 8);
            expect(asked == Session::ArenaBytes(8) && Close(s.infer(8, x.storage.data()), BiasProduct(x.logical, 8, false)), "the same Session without strides asks for the planned arena only");
         }
      }
   } catch (const std::exception &e) {
      out << "FAIL exception: " << e.what() << "\n";
      ++failures;
   }
   if (helper)
      sofie_hip_ctx_destroy(helper);
   std::strncpy(report, out.str().c_str(), len - 1);
   report[len - 1] = 0;
   return failures;
}
