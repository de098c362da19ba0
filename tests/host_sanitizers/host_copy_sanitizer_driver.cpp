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
  printf("ok: %d scatter/gather pairs under the sanitizers\n", runs);
  return 0;
}
