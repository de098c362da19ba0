// Host-only sanitizer run of the SSD engine: random layouts and id lists, both
// engines, both request modes; files vs a straightforward per-chunk model.
#include "fkv_ssd.cpp"
#include "fkv_ranges.cpp"
#include <random>
#include <cassert>
namespace fkv {
int fail(int code, const char *fmt, ...) { va_list ap; va_start(ap, fmt); vfprintf(stderr, fmt, ap); va_end(ap); fputc('\n', stderr); return code; }
void clear_error() {}
int caught(const char *where) noexcept { fprintf(stderr, "%s: exception\n", where); return 2; }
}
int main() {
  std::mt19937_64 rng(7);
  std::string base = std::string(getenv("TMPDIR") ? getenv("TMPDIR") : "/tmp") + "/fkv_asan_XXXXXX";
  std::vector<char> dirbuf(base.begin(), base.end()); dirbuf.push_back(0);
  char *dir = dirbuf.data();
  if (!mkdtemp(dir)) return 2;
  int runs = 0;
  for (int iter = 0; iter < 60; ++iter) {
    const int ndev = 1 + rng() % 2, nfiles = 1 + rng() % 3, rr = 1 + rng() % 3;
    const int layers = 1 + rng() % 5, kv = 1 + rng() % 2;
    const int64_t chunk = (1 + rng() % 64) * 512;
    const bool blockfirst = rng() % 2;
    const int ncpu = 8 + rng() % 24, nssd_per_file = 4 + rng() % 12;
    const int nssd = nssd_per_file * ndev * nfiles;
    int64_t cl, ck, cb, sl, sk;
    if (blockfirst) { ck = chunk; cl = kv * chunk; cb = layers * kv * chunk; sl = cl; sk = ck; }
    else { cb = chunk; ck = ncpu * chunk; cl = kv * ncpu * chunk; sk = nssd_per_file * chunk; sl = kv * nssd_per_file * chunk; }
    const int64_t pool_bytes = (int64_t)ncpu * layers * kv * chunk, file_bytes = (int64_t)nssd_per_file * layers * kv * chunk;
    std::vector<uint8_t> pool(pool_bytes), back(pool_bytes, 0);
    for (auto &b : pool) b = (uint8_t)rng();
    std::vector<std::string> paths; std::vector<const char *> cpaths;
    for (int i = 0; i < ndev * nfiles; ++i) {
      paths.push_back(std::string(dir) + "/f" + std::to_string(iter) + "_" + std::to_string(i));
      int fd = open(paths.back().c_str(), O_CREAT | O_RDWR | O_TRUNC, 0600); if (fd < 0 || ftruncate(fd, file_bytes)) return 3; close(fd);
    }
    for (auto &p : paths) cpaths.push_back(p.c_str());
    
    std::vector<int64_t> sid, cid(ncpu);
    for (int i = 0; i < nssd; ++i)   // ids whose place lies inside the files (striping with rr may not divide evenly)
      if (locate(i, rr, ndev, nfiles).in_file < nssd_per_file) sid.push_back(i);
    for (int i = 0; i < ncpu; ++i) cid[i] = i;
    const int n = 1 + rng() % std::min<int>(ncpu, (int)sid.size());
    std::shuffle(sid.begin(), sid.end(), rng); std::shuffle(cid.begin(), cid.end(), rng);
    if (rng() % 3 == 0) { std::sort(sid.begin(), sid.begin() + n); std::sort(cid.begin(), cid.begin() + n); }
    for (int entries : {0, 8}) for (int opt : {0, 1}) {
      fkv_ssd_ctx *ctx = nullptr;
      if (fkv_ssd_open(cpaths.data(), ndev, nfiles, entries, 0, &ctx)) return 4;
      if (fkv_ssd_transfer(ctx, 0, layers, pool.data(), sid.data(), cid.data(), n, cl, ck, sl, sk, chunk, cb, 0, rr, 3, kv, opt)) return 5;
      std::fill(back.begin(), back.end(), 0);
      if (fkv_ssd_transfer(ctx, 0, layers, back.data(), sid.data(), cid.data(), n, cl, ck, sl, sk, chunk, cb, 1, rr, 3, kv, opt)) return 6;
      for (int i = 0; i < n; ++i) for (int l = 0; l < layers; ++l) for (int k = 0; k < kv; ++k) {
        const int64_t off = cid[i] * cb + l * cl + k * ck;
        if (memcmp(pool.data() + off, back.data() + off, chunk)) { fprintf(stderr, "mismatch iter %d entries %d opt %d ndev %d nfiles %d rr %d layers %d kv %d chunk %lld blockfirst %d ncpu %d nssd_per_file %d n %d at i=%d l=%d k=%d sid %lld cid %lld\n", iter, entries, opt, ndev, nfiles, rr, layers, kv, (long long)chunk, (int)blockfirst, ncpu, nssd_per_file, n, i, l, k, (long long)sid[i], (long long)cid[i]); fkv_ssd_close(ctx); return 7; }
      }
      // plan dump stays inside its buffer
      std::vector<int64_t> rows(5 * 16);
      const int64_t r = fkv_ssd_plan(ndev, nfiles, 0, layers, sid.data(), cid.data(), n, cl, ck, sl, sk, chunk, cb, rr, kv, opt, rows.data(), 16);
      if (r < 0) return 8;
      fkv_ssd_close(ctx); ++runs;
    }
    for (auto &p : paths) unlink(p.c_str());
  }
  rmdir(dir);
  printf("ok: %d transfers round-tripped under the sanitizers\n", runs);
  return 0;
}
