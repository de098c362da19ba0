#include "fkv_host_copy.cpp"
#include <random>
#include <vector>
#include <cstdio>
#include <cstring>
#include <algorithm>
int main() {
  std::mt19937_64 rng(3);
  int runs = 0;
  for (int iter = 0; iter < 400; ++iter) {
    const int nblk = 1 + rng() % 40, nhost = nblk + rng() % 20;
    const int64_t chunk = 1 + rng() % 5000;
    const bool adjacent = rng() % 3 == 0;
    const int64_t stride = adjacent ? chunk : chunk + rng() % 300;
    const int threads = rng() % 5; const bool streaming = rng() % 2;
    const size_t mis = rng() % 64; // misaligned bases
    std::vector<uint8_t> staging(mis + (size_t)nblk * chunk), host(mis + (size_t)nhost * stride + chunk, 0xEE), ref;
    for (auto &b : staging) b = (uint8_t)rng();
    std::vector<int64_t> ids(nhost);
    for (int i = 0; i < nhost; ++i) ids[i] = i;
    std::shuffle(ids.begin(), ids.end(), rng);
    if (rng() % 2) std::sort(ids.begin(), ids.begin() + nblk);
    ref = host;
    for (int k = 0; k < nblk; ++k) memcpy(ref.data() + mis + ids[k] * stride, staging.data() + mis + (size_t)k * chunk, chunk);
    fkv::host_rows_copy(staging.data() + mis, host.data() + mis, ids.data(), nblk, stride, chunk, true, adjacent, threads, streaming);
    fkv::host_copy_fence(streaming);
    if (host != ref) { fprintf(stderr, "scatter mismatch iter %d\n", iter); return 1; }
    std::vector<uint8_t> back(staging.size(), 0);
    fkv::host_rows_copy(back.data() + mis, host.data() + mis, ids.data(), nblk, stride, chunk, false, adjacent, threads, streaming);
    fkv::host_copy_fence(streaming);
    if (memcmp(back.data() + mis, staging.data() + mis, (size_t)nblk * chunk)) { fprintf(stderr, "gather mismatch iter %d\n", iter); return 2; }
    ++runs;
  }
  // Rows of a batch gathered into a dense buffer by a crew that outlives the calls
  // (the host half of a gathered layerwise restore): pieces with two levels of strides.
  int gathers = 0;
  for (int helpers : {0, 1, 3}) {
    fkv::HostCrew crew(helpers);
    for (int iter = 0; iter < 100; ++iter) {
      const int rows = 1 + rng() % 60, pool = rows + rng() % 30;
      const int outer = 1 + rng() % 4, inner = 1 + rng() % 2;
      const int64_t piece = 1 + rng() % 3000;
      const int64_t inner_stride = piece + rng() % 100, outer_stride = inner * inner_stride + rng() % 200;
      const int64_t row_stride = outer * outer_stride + rng() % 500;
      const size_t mis = rng() % 64;
      std::vector<uint8_t> host(mis + (size_t)pool * row_stride + outer_stride), dense(mis + (size_t)rows * outer * inner * piece + 1, 0xAB);
      for (auto &b : host) b = (uint8_t)rng();
      std::vector<int64_t> ids(rows);
      for (auto &x : ids) x = rng() % pool; // duplicates allowed
      std::vector<uint8_t> want = dense;
      for (int r = 0; r < rows; ++r)
        for (int o = 0; o < outer; ++o)
          for (int i = 0; i < inner; ++i)
            memcpy(want.data() + mis + (((size_t)r * outer + o) * inner + i) * piece,
                   host.data() + mis + ids[r] * row_stride + o * outer_stride + i * inner_stride, piece);
      fkv::host_gather_rows(crew, dense.data() + mis, host.data() + mis, ids.data(), rows, row_stride,
                            outer, outer_stride, inner, inner_stride, piece);
      if (dense != want) { fprintf(stderr, "gather_rows mismatch helpers %d iter %d\n", helpers, iter); return 3; }
      ++gathers;
    }
  }
  printf("ok: %d scatter/gather pairs and %d crew gathers under the sanitizers\n", runs, gathers);
  return 0;
}
