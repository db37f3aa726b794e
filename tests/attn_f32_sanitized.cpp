// Address- and undefined-behaviour-sanitized run of the fp32 attention routines (vexact_amd/csrc/attn_f32.h) over
// random packed and paged batches with exactly sized heap buffers: any access outside a tensor aborts the run.
// (Values are checked against the oracle in tests/test_attn_f32_host.py; this run is about addresses.)
// Compiled and run by tests/test_attn_f32_host.py; nothing in the product uses it.
#define __host__
#define __device__
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "../vexact_amd/csrc/attn_f32.h"

int main() {
  std::mt19937_64 rng(777);
  auto rnd = [&](int64_t lo, int64_t hi) { return lo + (int64_t)(rng() % (uint64_t)(hi - lo + 1)); };
  auto fill = [&](std::vector<float>& v) { for (auto& x : v) x = (float)rnd(-1000, 1000) * 1e-3f; };
  for (int it = 0; it < 120; it++) {
    const int B = (int)rnd(1, 4), Hkv = (int)rnd(1, 3), G = (int)rnd(1, 3), Hq = Hkv * G;
    const int dk = (int)rnd(1, 40), dv = (int)rnd(1, 40), page = (int)rnd(1, 9);
    const bool paged = it % 2 == 0;
    std::vector<int> cu_q(B + 1, 0), cu_k(B + 1, 0), used(B), qlen(B), klen(B);
    for (int s = 0; s < B; s++) {
      qlen[s] = (int)rnd(0, 7);
      klen[s] = (int)rnd(0, 20);
      cu_q[s + 1] = cu_q[s] + qlen[s];
      cu_k[s + 1] = cu_k[s] + klen[s];
      used[s] = klen[s];
    }
    const int T = cu_q[B], Tk = cu_k[B];
    if (T == 0) continue;
    std::vector<float> q((size_t)T * Hq * dk), o((size_t)T * Hq * dv, 5.f), lse((size_t)T * Hq, 5.f);
    fill(q);
    vx::AttnF32 p = {};
    p.q = q.data(); p.sqt = (int64_t)Hq * dk; p.sqh = dk;
    p.o = o.data(); p.sot = (int64_t)Hq * dv; p.soh = dv;
    p.lse = lse.data();
    p.cu_q = cu_q.data();
    p.Hq = Hq; p.Hkv = Hkv; p.num_seqs = B; p.dk = dk; p.dv = dv; p.causal = (int)rnd(0, 4) != 0; p.scale = 0.3f;
    std::vector<float> k, v;
    std::vector<int> table;
    if (paged) {
      int maxp = 1, total_pages = 1;
      for (int s = 0; s < B; s++) {
        const int np = (klen[s] + page - 1) / page;
        maxp = np > maxp ? np : maxp;
        total_pages += np;
      }
      table.assign((size_t)B * maxp, -1);
      int next = 0;
      for (int s = 0; s < B; s++)
        for (int pg = 0; pg < (klen[s] + page - 1) / page; pg++) table[(size_t)s * maxp + pg] = next++;
      k.resize((size_t)total_pages * page * Hkv * dk);
      v.resize((size_t)total_pages * page * Hkv * dv);
      p.skb = (int64_t)page * Hkv * dk; p.skp = (int64_t)Hkv * dk; p.skh = dk;
      p.svb = (int64_t)page * Hkv * dv; p.svp = (int64_t)Hkv * dv; p.svh = dv;
      p.block_table = table.data(); p.bt_stride = maxp; p.page_size = page; p.max_kv = maxp * page;
      p.seqused_k = used.data();
      p.causal = 1;
      if (rnd(0, 3) == 0) used[(size_t)rnd(0, B - 1)] = 1000;  // a wrong length is clamped to what the table addresses
    } else {
      k.resize((size_t)(Tk > 0 ? Tk : 1) * Hkv * dk);
      v.resize((size_t)(Tk > 0 ? Tk : 1) * Hkv * dv);
      p.skp = (int64_t)Hkv * dk; p.skh = dk; p.svp = (int64_t)Hkv * dv; p.svh = dv;
      p.cu_k = cu_k.data(); p.packed = 1;
    }
    fill(k); fill(v);
    p.k = k.data(); p.v = v.data();
    for (int64_t idx = 0; idx < (int64_t)T * Hq; idx++) vx::attn_f32_forward_row(p, (int)(idx / Hq), (int)(idx % Hq));
    if (paged || !p.causal || Tk == 0) continue;
    // backward over the same packed batch
    std::vector<float> d_o((size_t)T * Hq * dv), delta((size_t)T * Hq), dq(q.size()), dkk((size_t)Tk * Hkv * dk), dvv((size_t)Tk * Hkv * dv);
    fill(d_o);
    for (int s = 0; s < B; s++)  // rows of a sequence without keys are left alone by the forward: give them a finite lse
      if (klen[s] == 0)
        for (int t = cu_q[s]; t < cu_q[s + 1]; t++)
          for (int h = 0; h < Hq; h++) lse[(size_t)t * Hq + h] = 0.f;
    vx::AttnF32Bwd b = {};
    b.q = q.data(); b.k = k.data(); b.v = v.data(); b.o = o.data(); b.d_o = d_o.data(); b.lse = lse.data(); b.delta = delta.data();
    b.dq = dq.data(); b.dk = dkk.data(); b.dv = dvv.data();
    b.sqt = p.sqt; b.sqh = p.sqh; b.skt = p.skp; b.skh = p.skh; b.svt = p.svp; b.svh = p.svh; b.sot = p.sot; b.soh = p.soh;
    b.sdt = p.sot; b.sdh = p.soh; b.sdqt = p.sqt; b.sdqh = p.sqh; b.sdkt = p.skp; b.sdkh = p.skh; b.sdvt = p.svp; b.sdvh = p.svh;
    b.cu_q = cu_q.data(); b.cu_k = cu_k.data(); b.Hq = Hq; b.Hkv = Hkv; b.num_seqs = B; b.dk_ = dk; b.dv_ = dv; b.scale = p.scale;
    for (int64_t idx = 0; idx < (int64_t)T * Hq; idx++) vx::attn_f32_delta_row(b, (int)(idx / Hq), (int)(idx % Hq));
    for (int64_t idx = 0; idx < (int64_t)T * Hq; idx++) vx::attn_f32_dq_row(b, (int)(idx / Hq), (int)(idx % Hq));
    for (int64_t idx = 0; idx < (int64_t)Tk * Hkv; idx++) vx::attn_f32_dkv_row(b, (int)(idx / Hkv), (int)(idx % Hkv));
  }
  std::puts("attn_f32 sanitized run ok");
  return 0;
}
