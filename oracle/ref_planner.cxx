// C entry point around the reference's own OrganizeMemory, which is included from the reference
// checkout at build time (nothing of it is copied here).  Test infrastructure only.
#include <algorithm>
#include <cstddef>
#include <set>
#include <stdexcept>
#include <unordered_map>
#include <vector>

#include REF_PLANNER_INC

extern "C" __attribute__((visibility("default"))) int ref_organize_memory(int n, const int *begin, const int *end,
                                                                          const std::size_t *size, std::size_t *offsets,
                                                                          std::size_t *total_bytes,
                                                                          std::size_t *total_free_bytes,
                                                                          std::size_t *largest_free_block)
{
   try {
      std::vector<TensorLifeInfo> info((std::size_t)n);
      for (int i = 0; i < n; ++i)
         info[(std::size_t)i] = TensorLifeInfo{begin[i], end[i], size[i]};
      MemoryResult r = OrganizeMemory(info);
      for (int i = 0; i < n; ++i)
         offsets[i] = r.offsets[(std::size_t)i];
      *total_bytes = r.total_bytes;
      *total_free_bytes = r.total_free_bytes;
      *largest_free_block = r.largest_free_block;
      return 0;
   } catch (const std::exception &) {
      return 1;
   }
}
