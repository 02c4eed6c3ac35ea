// sampling_server: same command line as the reference binary
//   sampling_server <gpu_number> <cache_agg_mode> <dyn_cache> [fanout, e.g. 25,10]
// (Legion-IBP sampling_server/src/main.cu:5-17).  Reads ./meta_config, builds the
// cache, serves `epoch` passes over the training set.  The reference hard-codes
// the fanout {25,10} and ignores its launcher's --fanout; the optional fourth
// argument supplies it here.
//
// LEGION_MI_DUMP=<dir> writes the first LEGION_MI_DUMP_BATCHES (default 2) batches
// to <dir>/batch_<i>.bin: node_counter[16], edge_counter[16], ids, agg_src_off,
// agg_dst_off, features -- for checking a deployment against the CPU oracle.
#include <cstdio>
#include <cstdlib>
#include <iostream>
#include <string>
#include <vector>

#include "legion_host.hpp"

namespace {
struct Dump {
  std::string dir;
  int left = 0, index = 0;
};

void dump_sink(const lmi_batch_view *b, int, int, void *stream, void *user) {
  Dump *d = (Dump *)user;
  if (d->left <= 0) return;
  lmi_stream_sync(stream);
  int32_t nc[16], ec[16];
  lmi_copy_to_host(nc, b->node_counter, 64);
  lmi_copy_to_host(ec, b->edge_counter, 64);
  const int hops = nc[8];
  const int64_t n = nc[9 + hops];
  int64_t e = 0;
  for (int k = 1; k <= hops; ++k) e += ec[9 + k];
  std::vector<int32_t> ids((size_t)n), src((size_t)e), dst((size_t)e);
  std::vector<unsigned char> feat((size_t)n * (size_t)b->row_bytes);  // fp32 or fp16 rows, as served
  if (n) lmi_copy_to_host(ids.data(), b->ids, (size_t)n * 4);
  if (e) lmi_copy_to_host(src.data(), b->agg_src_off, (size_t)e * 4);
  if (e) lmi_copy_to_host(dst.data(), b->agg_dst_off, (size_t)e * 4);
  if (n) lmi_copy_to_host(feat.data(), b->features, feat.size());
  const std::string path = d->dir + "/batch_" + std::to_string(d->index) + ".bin";
  FILE *f = std::fopen(path.c_str(), "wb");
  if (f) {
    std::fwrite(nc, 4, 16, f);
    std::fwrite(ec, 4, 16, f);
    std::fwrite(ids.data(), 4, ids.size(), f);
    std::fwrite(src.data(), 4, src.size(), f);
    std::fwrite(dst.data(), 4, dst.size(), f);
    std::fwrite(feat.data(), 1, feat.size(), f);
    std::fclose(f);
  }
  --d->left;
  ++d->index;
}
}  // namespace

int main(int argc, char **argv) {
  if (argc < 4) {
    std::fprintf(stderr, "usage: %s <gpu_number> <cache_agg_mode> <dyn_cache> [fanout,fanout,...]\n", argv[0]);
    return 2;
  }
  std::cout << "Start Sampling Server\n";
  std::vector<int> fanout;
  if (argc > 4) {
    std::string s = argv[4];
    size_t pos = 0;
    while (pos < s.size()) {
      size_t c = s.find(',', pos);
      if (c == std::string::npos) c = s.size();
      fanout.push_back(std::atoi(s.substr(pos, c - pos).c_str()));
      pos = c + 1;
    }
  } else {
    fanout = {25, 10};
  }
  Server *server = NewGPUServer();
  std::cout << "Dynamic? " << std::atoi(argv[3]) << "\n";
  server->Initialize(std::atoi(argv[1]), fanout, 1, std::atoi(argv[3]));
  Dump dump;
  if (const char *dir = std::getenv("LEGION_MI_DUMP")) {
    dump.dir = dir;
    const char *nb = std::getenv("LEGION_MI_DUMP_BATCHES");
    dump.left = nb ? std::atoi(nb) : 2;
    server->SetBatchSink(dump_sink, &dump);
  }
  server->PreSc(std::atoi(argv[2]));
  server->Run();
  server->Finalize();
  delete server;
  return 0;
}
