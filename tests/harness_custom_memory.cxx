// Test harness for Sessions emitted with Options::kCustomMemory: the scenarios of the reference's
// tests/alpaka/TestAlpakaCustomMemory.cxx (one block allocated and assigned, assign optional, a null assignment and a
// missing alloc are rejected, custom memory together with an external stream), driven from Python through one C function.
// The device block comes from a second runtime context's arena, so this file needs no HIP header.
#include "CustomMemoryChain_GPU_HIP.hxx"
#include "CustomMemoryStreamChain_GPU_HIP.hxx"
#include "CustomMemoryDynamicChain_GPU_HIP.hxx"

#include <cmath>
#include <cstdio>
#include <cstring>
#include <set>
#include <sstream>

namespace {
struct State {
   int allocations = 0, deallocations = 0;
   std::size_t blockBytes = 0;
   char *block = nullptr;
   std::vector<std::size_t> offsets;
};

template <class Provider>
Provider MakeProvider(State &st, char *memory, bool withAssign)
{
   Provider p;
   p.alloc = [&st, memory](std::size_t bytes) -> void * {
      ++st.allocations;
      st.blockBytes = bytes;
      st.block = memory;
      return memory;
   };
   p.dealloc = [&st](void *) { ++st.deallocations; };
   if (withAssign)
      p.assign = [&st](std::size_t off) -> void * {
         st.offsets.push_back(off);
         return st.block + off;
      };
   return p;
}

bool ChainOk(const std::vector<float> &y)
{
   const float want = std::tanh(1.f / (1.f + std::exp(-3.5f)));
   if (y.size() != 12)
      return false;
   for (float v : y)
      if (std::fabs(v - want) > 1e-5f)
         return false;
   return true;
}
} // namespace

extern "C" int run_custom_memory(const char *dir, char *report, int len)
{
   std::ostringstream out;
   int failures = 0;
   auto expect = [&](bool ok, const char *what) {
      out << (ok ? "ok " : "FAIL ") << what << "\n";
      failures += ok ? 0 : 1;
   };
   sofie_hip_ctx *helper = nullptr;
   try {
      if (sofie_hip_ctx_create(&helper, 0, nullptr) || sofie_hip_arena_create(helper, 1 << 20, 256))
         throw std::runtime_error(sofie_hip_last_error());
      char *memory = static_cast<char *>(sofie_hip_arena_ptr(helper, 4096));
      const std::string w1 = std::string(dir) + "/CustomMemoryChain_GPU_HIP.dat", w2 = std::string(dir) + "/CustomMemoryStreamChain_GPU_HIP.dat";
      std::vector<float> ones(15, 1.f);
      {
         using namespace SOFIE_CustomMemoryChain;
         State st;
         {
            Session s(MakeProvider<MemoryProvider>(st, memory, true), w1);
            expect(st.allocations == 1 && st.deallocations == 0, "one block allocated");
            expect(st.blockBytes == Session::kArenaBytes && st.blockBytes <= (1u << 20) - 4096, "block size is the planned arena");
            bool aligned = st.offsets.size() >= 4;
            for (std::size_t o : st.offsets)
               aligned = aligned && o % 256 == 0 && o < st.blockBytes;
            expect(aligned, "every tensor assigned at a 256-byte offset inside the block");
            expect(std::set<std::size_t>(st.offsets.begin(), st.offsets.end()).size() >= 3, "distinct offsets");
            expect(ChainOk(s.infer(ones.data())), "chain result with assign");
            expect(reinterpret_cast<char *>(s.device_input_X()) >= memory && reinterpret_cast<char *>(s.device_input_X()) < memory + st.blockBytes,
                   "tensors live in the caller's block");
         }
         expect(st.deallocations == 1, "block returned once");
         State st2;
         {
            Session s(MakeProvider<MemoryProvider>(st2, memory, false), w1);
            expect(st2.allocations == 1, "assign is optional: one allocation");
            expect(ChainOk(s.infer(ones.data())), "chain result without assign");
         }
         expect(st2.deallocations == 1, "assign is optional: block returned");
         State st3;
         auto bad = MakeProvider<MemoryProvider>(st3, memory, true);
         bad.assign = [](std::size_t) -> void * { return nullptr; };
         bool threw = false;
         try {
            Session s(bad, w1);
         } catch (const std::runtime_error &) {
            threw = true;
         }
         expect(threw && st3.deallocations == 1, "a null assignment is rejected and the block returned");
         threw = false;
         try {
            Session s(MemoryProvider{}, w1);
         } catch (const std::runtime_error &) {
            threw = true;
         }
         expect(threw, "a provider without alloc is rejected");
      }
      {
         using namespace SOFIE_CustomMemoryStreamChain;
         State st;
         {
            Session s(MakeProvider<MemoryProvider>(st, memory, true), w2, sofie_hip_stream(helper));
            expect(s.stream() == sofie_hip_stream(helper), "the caller's stream is used");
            expect(ChainOk(s.infer(ones.data())), "chain result on the caller's stream");
         }
         expect(st.allocations == 1 && st.deallocations == 1, "external stream and custom memory: one block, returned");
      }
      {
         // run-time batch + caller's memory + caller's stream + safetensors weights in one Session
         using namespace SOFIE_CustomMemoryDynamicChain;
         const std::string w3 = std::string(dir) + "/CustomMemoryDynamicChain_GPU_HIP.safetensors";
         const float want = std::tanh(1.f / (1.f + std::exp(-3.5f)));
         auto rowsOk = [&](const std::vector<float> &y, std::size_t rows) {
            bool ok = y.size() == rows * 4;
            for (float v : y)
               ok = ok && std::fabs(v - want) <= 1e-5f;
            return ok;
         };
         State st;
         {
            Session s(MakeProvider<MemoryProvider>(st, memory, true), w3, 7, sofie_hip_stream(helper));
            expect(st.allocations == 1 && st.blockBytes == Session::ArenaBytes(7) && st.blockBytes == Session::ArenaBytes(16) &&
                      Session::ArenaBytes(17) > st.blockBytes,
                   "run-time batch: the block is the static part plus 16 batch entries");
            bool aligned = !st.offsets.empty();
            for (std::size_t o : st.offsets)
               aligned = aligned && o % 256 == 0 && o < st.blockBytes;
            expect(aligned, "run-time batch: every tensor assigned at a 256-byte offset inside the block");
            std::vector<float> x(7 * 5, 1.f);
            expect(rowsOk(s.infer(7, x.data()), 7), "run-time batch: 7 rows");
            expect(rowsOk(s.infer(2, x.data()), 2), "run-time batch: 2 rows on the same session");
            bool threw = false;
            try {
               s.infer(8, x.data());
            } catch (const std::runtime_error &) {
               threw = true;
            }
            expect(threw, "run-time batch: more than the maximum is refused");
            expect(s.stream() == sofie_hip_stream(helper) && s.GetMaxBatch() == 7, "run-time batch: caller's stream, maximum kept");
         }
         expect(st.deallocations == 1, "run-time batch: block returned once");
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
