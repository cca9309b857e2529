// Placement of intermediate tensors into one arena.  Same policy and same result as the reference's
// OrganizeMemory (core/inc/SOFIE/utils/shared/MemoryPlanner.inc:33-132): tensor i lives in [begin, end);
// sweep the events in time order, frees before allocations at equal times; an allocation takes the
// smallest free block that fits (lowest offset among equals) from its start, else the pool grows; freed
// blocks merge with their neighbours.  Events with equal (time, kind) are taken in tensor order.
#ifndef SOFIE_HIP_MEMORYPLANNER
#define SOFIE_HIP_MEMORYPLANNER

#include <algorithm>
#include <cstddef>
#include <stdexcept>
#include <vector>

namespace SOFIE_HIP {

struct TensorLifeInfo {
   int begin;
   int end;
   std::size_t size;
};

struct MemoryResult {
   std::size_t total_bytes = 0;
   std::vector<std::size_t> offsets;
   std::size_t total_free_bytes = 0;
   std::size_t largest_free_block = 0;
};

inline MemoryResult OrganizeMemory(const std::vector<TensorLifeInfo> &tensors)
{
   struct Event {
      int t, kind, idx;
   };
   struct Block {
      std::size_t off, size;
   };
   for (const auto &t : tensors)
      if (!(t.end > t.begin))
         throw std::runtime_error("Each tensor must have end > begin.");
   std::vector<Event> events;
   for (int i = 0; i < (int)tensors.size(); ++i) {
      events.push_back({tensors[i].end, 0, i});
      events.push_back({tensors[i].begin, 1, i});
   }
   std::sort(events.begin(), events.end(), [](const Event &a, const Event &b) {
      if (a.t != b.t)
         return a.t < b.t;
      if (a.kind != b.kind)
         return a.kind < b.kind;
      return a.idx < b.idx;
   });
   MemoryResult r;
   r.offsets.assign(tensors.size(), 0);
   std::vector<Block> free_list; // sorted by offset
   std::vector<char> live(tensors.size(), 0);
   for (const auto &e : events) {
      if (e.kind == 0) {
         if (!live[e.idx])
            continue;
         live[e.idx] = 0;
         Block fb{r.offsets[e.idx], tensors[e.idx].size};
         auto pos = std::lower_bound(free_list.begin(), free_list.end(), fb, [](const Block &a, const Block &b) { return a.off < b.off; });
         pos = free_list.insert(pos, fb);
         if (pos != free_list.begin() && (pos - 1)->off + (pos - 1)->size == pos->off) {
            (pos - 1)->size += pos->size;
            pos = free_list.erase(pos) - 1;
         }
         if (pos + 1 != free_list.end() && pos->off + pos->size == (pos + 1)->off) {
            pos->size += (pos + 1)->size;
            free_list.erase(pos + 1);
         }
      } else {
         const std::size_t need = tensors[e.idx].size;
         int best = -1;
         for (int i = 0; i < (int)free_list.size(); ++i)
            if (free_list[i].size >= need && (best < 0 || free_list[i].size < free_list[best].size))
               best = i;
         const std::size_t before = r.total_bytes;
         std::size_t off;
         if (best >= 0) {
            off = free_list[best].off;
            if (free_list[best].size == need) {
               free_list.erase(free_list.begin() + best);
            } else {
               free_list[best].off += need;
               free_list[best].size -= need;
            }
         } else {
            off = r.total_bytes;
            r.total_bytes += need;
         }
         r.offsets[e.idx] = off;
         live[e.idx] = 1;
         if (r.total_bytes > before) {
            r.total_free_bytes = 0;
            r.largest_free_block = 0;
            for (const auto &fb : free_list) {
               r.total_free_bytes += fb.size;
               r.largest_free_block = std::max(r.largest_free_block, fb.size);
            }
         }
      }
   }
   return r;
}

} // namespace SOFIE_HIP
#endif
