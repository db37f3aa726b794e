// Address- and undefined-behaviour-sanitized run of the host-side step metadata builder and block allocator
// (vexact_amd/csrc/host_meta.cpp) on random steps with exactly sized heap buffers: any read or write outside a buffer
// aborts the run. Compiled and run by tests/test_host_logic.py; nothing in the product uses it.
#include <cstdio>
#include <cstdlib>
#include <random>

#include "../vexact_amd/csrc/host_meta.cpp"

#define CHECK(c) do { if (!(c)) { std::fprintf(stderr, "check failed at line %d: %s\n", __LINE__, #c); std::exit(1); } } while (0)

int main() {
  std::mt19937_64 rng(12345);
  auto rnd = [&](int64_t lo, int64_t hi) { return lo + (int64_t)(rng() % (uint64_t)(hi - lo + 1)); };
  for (int it = 0; it < 400; it++) {
    const int32_t page = (int32_t)rnd(1, 33);
    const int64_t n = rnd(0, 12), max_blocks = rnd(1, 20);
    std::vector<int64_t> done((size_t)n), step((size_t)n), off((size_t)n + 1, 0);
    std::vector<int32_t> ids;
    int64_t total = 0;
    for (int64_t s = 0; s < n; s++) {
      const int64_t nb = rnd(0, max_blocks);
      done[(size_t)s] = nb == 0 ? 0 : rnd(0, nb * page);
      step[(size_t)s] = rnd(0, std::min<int64_t>(done[(size_t)s], 9));
      total += step[(size_t)s];
      for (int64_t b = 0; b < nb; b++) ids.push_back((int32_t)rnd(0, 4095));
      off[(size_t)s + 1] = (int64_t)ids.size();
    }
    const bool fits = rnd(0, 9) != 0;  // one in ten buckets is too small: must be refused without a write
    // buckets hold at least one token and one sequence (the entry point refuses null output pointers)
    const int64_t cap_tokens = fits ? total + rnd(total == 0 ? 1 : 0, 5) : std::max<int64_t>(total - 1, 1);
    const int64_t cap_seqs = std::max<int64_t>(n + rnd(0, 3), 1);
    std::vector<int64_t> positions((size_t)cap_tokens, -7);
    std::vector<int32_t> slots((size_t)cap_tokens, -7), qsl((size_t)cap_seqs + 1, -7), ctx((size_t)cap_seqs, -7),
        tables((size_t)(cap_seqs * max_blocks), -7), order((size_t)cap_seqs, -7);
    int64_t tot = -1;
    int32_t maxq = -1;
    const int rc = vx_host_step_metadata(n, done.data(), step.data(), ids.empty() ? (const int32_t*)&page : ids.data(), off.data(), page,
                                         max_blocks, cap_tokens, cap_seqs, positions.data(), slots.data(), qsl.data(), ctx.data(),
                                         tables.data(), order.data(), &tot, &maxq);
    if (!fits && total > cap_tokens) {
      CHECK(rc == VX_ERR_ARG);
      continue;
    }
    CHECK(rc == VX_OK && tot == total);
    int64_t i = 0;
    for (int64_t s = 0; s < n; s++) {
      CHECK(qsl[(size_t)s] == (int32_t)i && ctx[(size_t)s] == (int32_t)done[(size_t)s]);
      for (int64_t pos = done[(size_t)s] - step[(size_t)s]; pos < done[(size_t)s]; pos++, i++) {
        CHECK(positions[(size_t)i] == pos);
        CHECK(slots[(size_t)i] == ids[(size_t)(off[(size_t)s] + pos / page)] * page + (int32_t)(pos % page));
      }
    }
    CHECK(qsl[(size_t)n] == (int32_t)total);
    for (; i < cap_tokens; i++) CHECK(positions[(size_t)i] == 0 && slots[(size_t)i] == -1);
    for (int64_t s = n; s < cap_seqs; s++) CHECK(qsl[(size_t)s + 1] == (int32_t)total && ctx[(size_t)s] == 0);
    for (int64_t s = 0; s + 1 < cap_seqs; s++) CHECK(ctx[(size_t)order[(size_t)s]] >= ctx[(size_t)order[(size_t)s + 1]]);
  }
  // allocator: random allocate / free traces against a bitmap, with double frees and foreign ids
  for (int it = 0; it < 50; it++) {
    const int64_t nblocks = rnd(0, 64);
    void* a = vx_kv_allocator_create(nblocks);
    CHECK(a);
    std::vector<uint8_t> used((size_t)nblocks, 0);
    int64_t free_n = nblocks;
    for (int op = 0; op < 200; op++) {
      if (rnd(0, 1)) {
        const int32_t page = (int32_t)rnd(1, 16);
        const int64_t cur = rnd(0, 4), tokens = rnd(0, 80);
        const int64_t need = std::max<int64_t>((tokens + page - 1) / page - cur, 0);
        std::vector<int32_t> out((size_t)need, -1);
        const int64_t got = vx_kv_allocator_allocate(a, tokens, cur, page, out.data(), need);
        if (need > free_n) {
          CHECK(got == -1);
        } else {
          CHECK(got == need);
          int64_t lowest = 0;
          for (int64_t k = 0; k < got; k++) {  // the lowest free ids, ascending
            while (used[(size_t)lowest]) lowest++;
            CHECK(out[(size_t)k] == (int32_t)lowest);
            used[(size_t)lowest] = 1;
          }
          free_n -= got;
        }
      } else {
        const int64_t m = rnd(0, 6);
        std::vector<int32_t> give((size_t)m);
        int64_t expect = 0;
        for (int64_t k = 0; k < m; k++) {
          give[(size_t)k] = (int32_t)rnd(-2, nblocks + 1);
          const int32_t b = give[(size_t)k];
          if (b >= 0 && b < nblocks && used[(size_t)b]) { used[(size_t)b] = 0; expect++; }
        }
        CHECK(vx_kv_allocator_free(a, give.data(), m) == expect);
        free_n += expect;
      }
      CHECK(vx_kv_allocator_num_free(a) == free_n);
    }
    vx_kv_allocator_destroy(a);
  }
  std::puts("host_meta sanitized run ok");
  return 0;
}
