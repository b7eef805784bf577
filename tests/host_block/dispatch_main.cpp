// Runs the dispatch functions of fta_device.h on the CPU, one host thread per GPU thread, for every
// workgroup id of a launch, and prints what each workgroup resolved. Input (stdin, one case per line):
//   bsz num_splits units row_blocks cache_len block_threads  len_0 .. len_{bsz-1}  bound_0 .. bound_15  chunk_0 .. chunk_15
// Output per case: one line "case <n>" and per workgroup id "<id> <live> <batch> <split> <len> <chunk> <unit> <row_block> <batch_chunk>".
#include <cstdio>
#include <iostream>
#include <sstream>
#include <string>

#include "fta_device.h"

int main() {
  std::string line;
  int case_no = 0;
  while (std::getline(std::cin, line)) {
    if (line.empty()) continue;
    std::istringstream in(line);
    fta::KernelParams p{};
    int threads;
    in >> p.bsz >> p.num_splits >> p.units >> p.row_blocks >> p.cache_len >> threads;
    std::vector<int64_t> lens(p.bsz);
    for (auto& v : lens) in >> v;
    for (int i = 0; i < FTA_LEN_BUCKETS; ++i) in >> p.len_bound[i];
    for (int i = 0; i < FTA_LEN_BUCKETS; ++i) in >> p.chunk_by_len[i];
    p.chunk = p.chunk_by_len[FTA_LEN_BUCKETS - 1];
    p.lens = lens.data();
    p.len_is_i64 = 1;
    std::printf("case %d\n", case_no++);
    const int grid = p.num_splits * p.units * p.bsz * p.row_blocks;
    int first_bchunk = -1;
    blockDim = dim3(threads);
    for (int id = 0; id < grid; ++id) {
      host_block::Block block(threads);
      host_block::current() = &block;
      struct Out { int live, batch, split, len, chunk, unit, row_block, bchunk; };
      std::vector<Out> outs(threads);
      std::vector<std::thread> pool;
      std::string error;
      for (int t = 0; t < threads; ++t)
        pool.emplace_back([&, t] {
          threadIdx = dim3(t);
          blockIdx = dim3(id);
          try {
            const fta::WorkItem w = fta::decode_work(p, id);
            Out o{};
            o.live = fta::item_by_order(p, w.item, &o.batch, &o.split, &o.len, &o.chunk) ? 1 : 0;
            o.unit = w.unit;
            o.row_block = w.row_block;
            outs[t] = o;
          } catch (const std::exception& e) {
            error = e.what();
            std::abort();
          }
        });
      for (auto& th : pool) th.join();
      // stage 2 derives the chunk by itself (a second kernel): run that function in a block of its own (the value
      // does not depend on the workgroup, so the first few ids stand for all)
      if (id >= 4) {
        for (int t = 1; t < threads; ++t)
          if (std::memcmp(&outs[t], &outs[0], sizeof(Out)) != 0) {
            std::printf("MISMATCH between threads of workgroup %d\n", id);
            return 1;
          }
        const Out& o = outs[0];
        std::printf("%d %d %d %d %d %d %d %d %d\n", id, o.live, o.batch, o.split, o.len, o.chunk, o.unit, o.row_block, first_bchunk);
        continue;
      }
      host_block::Block block2(256);
      host_block::current() = &block2;
      blockDim = dim3(256);
      std::vector<int> bchunk(256);
      pool.clear();
      for (int t = 0; t < 256; ++t)
        pool.emplace_back([&, t] {
          threadIdx = dim3(t);
          bchunk[t] = fta::batch_chunk(p);
        });
      for (auto& th : pool) th.join();
      blockDim = dim3(threads);
      for (int t = 1; t < threads; ++t)
        if (std::memcmp(&outs[t], &outs[0], sizeof(Out)) != 0) {
          std::printf("MISMATCH between threads of workgroup %d\n", id);
          return 1;
        }
      for (int t = 1; t < 256; ++t)
        if (bchunk[t] != bchunk[0]) {
          std::printf("MISMATCH of batch_chunk between threads\n");
          return 1;
        }
      first_bchunk = bchunk[0];
      const Out& o = outs[0];
      std::printf("%d %d %d %d %d %d %d %d %d\n", id, o.live, o.batch, o.split, o.len, o.chunk, o.unit, o.row_block, bchunk[0]);
    }
  }
  return 0;
}
