// Work lists of the prefill attention kernel (see prefill_plan.cpp).
#pragma once

#include <stdint.h>

#include <vector>

namespace me {

struct WorkList {
  std::vector<int32_t> work;          // 8 ints per entry: item, first token, tokens, first position, first key,
                                      // last key, chunk or -1, 1 if its bundle ends with it
  std::vector<int32_t> bundle_first;  // the first entry of each bundle
  std::vector<int32_t> token_chunks;  // per token: into how many chunks its tile's keys are cut
  int max_chunks = 1;
};

bool wide_blocks_pay(const int* starts, const int* qlens, int items, int tpb, int window, int nkv, int slots);
void build_work_list(const int* starts, const int* qlens, int items, int tpb, int window, int nkv, int slots,
                     long long partial_row_bytes, WorkList& out);

}  // namespace me
