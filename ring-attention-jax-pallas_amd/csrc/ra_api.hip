// C ABI of the ring-attention block-step library: argument validation (host only, before
// any HIP call) and dispatch to the gfx950 kernels.
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <vector>

#include "ra_launch.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int hip_fail(hipError_t e, const char* what) {
  return fail(RA_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// The kernels reach the rows that one wave moves (up to 16 of them) through an unsigned 32-bit byte
// offset per lane from the wave's first row: rows may not overlap and the row stride stays below 2^27.
constexpr int64_t kMaxRowStride = RA_MAX_ROW_STRIDE;

int check_tensor(const char* name, const ra_tensor& t, int D) {
  if (!t.ptr) return fail(RA_ERR_NULL, "%s.ptr is NULL", name);
  if (!aligned16(t.ptr)) return fail(RA_ERR_ALIGN, "%s.ptr is not 16-byte aligned", name);
  if ((t.stride_b % 8) || (t.stride_h % 8) || (t.stride_l % 8))
    return fail(RA_ERR_ALIGN, "%s strides must be multiples of 8 elements (16 bytes)", name);
  if (t.stride_l < D || t.stride_l > kMaxRowStride)
    return fail(RA_ERR_SHAPE, "%s.stride_l = %lld: the row stride must lie in [D, 2^27] elements", name,
                (long long)t.stride_l);
  return RA_OK;
}

// Token positions (offset + index) stay below 2^30 - 2^16 and the window is clamped to 2^30: every
// position difference, with a window and a tile added, then fits 32 bits in the kernels.
constexpr int64_t kMaxPos = ((int64_t)1 << 30) - (1 << 16);
constexpr int kMaxWindow = 1 << 30;  // wider than any position difference: masks nothing more
constexpr int kMaxLen = 1 << 24;
constexpr int kMaxSegLen = 65536;  // tile-list capacity of the kernels (1024 tiles x 64)

int check_dims(int B, int H, int Lq, int Lk, int D) {
  if (B <= 0 || H <= 0 || Lq <= 0 || Lk <= 0)
    return fail(RA_ERR_SHAPE, "B, H, Lq, Lk must be positive (got %d, %d, %d, %d)", B, H, Lq, Lk);
  if (Lq > kMaxLen || Lk > kMaxLen)
    return fail(RA_ERR_SHAPE, "shard length above %d tokens", kMaxLen);
  if ((int64_t)B * H > (1 << 20)) return fail(RA_ERR_SHAPE, "B*H too large");
  // the smallest tile any kernel hands to a workgroup is 128 tokens: the flat grid of the launch
  // must fit the 31 bits of a grid dimension
  const int64_t tiles = ((int64_t)(Lq > Lk ? Lq : Lk) + 127) / 128;
  if ((int64_t)B * H * tiles > 0x7fffffffll)
    return fail(RA_ERR_SHAPE, "B*H*ceil(L/128) = %lld workgroups exceed the grid limit of 2^31-1",
                (long long)((int64_t)B * H * tiles));
  if (D != 64 && D != 128) return fail(RA_ERR_HEAD_DIM, "head dim %d unsupported (64 or 128)", D);
  return RA_OK;
}

int check_bias(const ra_bias& b, int Lq, int Lk) {
  const int known = RA_BIAS_CAUSAL | RA_BIAS_WINDOW | RA_BIAS_SEGMENT | RA_BIAS_PREFIX | RA_BIAS_ALIBI |
                    RA_BIAS_DENSE;
  if (b.flags & ~known) return fail(RA_ERR_BIAS, "unknown bias flag bits 0x%x", b.flags & ~known);
  if ((b.flags & RA_BIAS_WINDOW) && b.window <= 0)
    return fail(RA_ERR_BIAS, "window must be positive (got %d)", b.window);
  if ((b.flags & RA_BIAS_CAUSAL) && (b.flags & RA_BIAS_PREFIX))
    return fail(RA_ERR_BIAS, "causal attention does not support a prefix mask");
  if ((b.flags & RA_BIAS_SEGMENT) && (!b.q_segment_ids || !b.kv_segment_ids))
    return fail(RA_ERR_NULL, "segment bias needs q_segment_ids and kv_segment_ids");
  if ((b.flags & RA_BIAS_SEGMENT) && (Lq > kMaxSegLen || Lk > kMaxSegLen))
    return fail(RA_ERR_SHAPE, "segment bias supports shards of at most %d tokens", kMaxSegLen);
  if ((b.flags & RA_BIAS_PREFIX) && (!b.q_prefix || !b.kv_prefix))
    return fail(RA_ERR_NULL, "prefix bias needs q_prefix and kv_prefix");
  if ((b.flags & RA_BIAS_ALIBI) && !b.alibi_slopes)
    return fail(RA_ERR_NULL, "ALiBi bias needs alibi_slopes");
  if (b.flags & RA_BIAS_DENSE) {
    if (!b.dense_bias) return fail(RA_ERR_NULL, "dense bias needs dense_bias");
    if (((uintptr_t)b.dense_bias & 3) != 0) return fail(RA_ERR_ALIGN, "dense_bias is not 4-byte aligned");
    if (b.dense_stride_q < Lk || b.dense_stride_b < 0 || b.dense_stride_h < 0)
      return fail(RA_ERR_BIAS, "dense bias strides: stride_q must be at least Lk, stride_b / stride_h "
                               "non-negative (0 broadcasts)");
    if (b.dense_map && (Lq > kMaxSegLen || Lk > kMaxSegLen))
      return fail(RA_ERR_SHAPE, "a dense bias with its summary supports shards of at most %d tokens", kMaxSegLen);
  }
  if (b.q_offset < 0 || b.kv_offset < 0 || b.q_offset + Lq > kMaxPos || b.kv_offset + Lk > kMaxPos)
    return fail(RA_ERR_BIAS, "token positions (offset + index) must lie in [0, 2^30 - 2^16)");
  return RA_OK;
}

ra::TensorArg to_arg(const ra_tensor& t) {
  return ra::TensorArg{(const ra::bf16_t*)t.ptr, t.stride_b, t.stride_h, t.stride_l};
}

ra::BiasArgs to_bias(const ra_bias& b) {
  ra::BiasArgs r;
  r.flags = b.flags;
  r.window = b.window < kMaxWindow ? b.window : kMaxWindow;
  r.q_off = (int)b.q_offset;
  r.kv_off = (int)b.kv_offset;
  r.q_seg = b.q_segment_ids;
  r.kv_seg = b.kv_segment_ids;
  r.q_seg_sb = b.q_segment_stride_b;
  r.kv_seg_sb = b.kv_segment_stride_b;
  r.q_pre = b.q_prefix;
  r.kv_pre = b.kv_prefix;
  r.q_pre_sb = b.q_prefix_stride_b;
  r.kv_pre_sb = b.kv_prefix_stride_b;
  r.slopes = b.alibi_slopes;
  r.dense = b.dense_bias;
  r.dense_sb = b.dense_stride_b;
  r.dense_sh = b.dense_stride_h;
  r.dense_sq = b.dense_stride_q;
  r.dense_map = (b.flags & RA_BIAS_DENSE) ? b.dense_map : nullptr;
  return r;
}

// kernel variant: 0 = causal / window only, 1 = per-tile terms, 2 = with a dense bias block
int kernel_mode(int flags) {
  if (flags & RA_BIAS_DENSE) return 2;
  return (flags & (RA_BIAS_SEGMENT | RA_BIAS_PREFIX | RA_BIAS_ALIBI)) != 0 ? 1 : 0;
}

constexpr float kLog2eHost = 1.4426950408889634f;

ra::BwdArgs to_bwd_args(const ra_bwd_step_params& p) {
  ra::BwdArgs a;
  a.q = to_arg(p.q);
  a.k = to_arg(p.k);
  a.v = to_arg(p.v);
  a.dout = to_arg(p.dout);
  a.lse = p.lse;
  a.delta = p.delta;
  a.dq = p.dq;
  a.dk = p.dk;
  a.dv = p.dv;
  a.B = p.B;
  a.H = p.H;
  a.Lq = p.Lq;
  a.Lk = p.Lk;
  a.scale2 = p.sm_scale * kLog2eHost;
  int e2 = 0;
  const float mant = frexpf(a.scale2, &e2);  // scale2 = mant * 2^e2, mant in [0.5, 1)
  a.scale_p2 = ldexpf(1.0f, e2 - 1);
  a.scale_res = mant * 2.0f;
  a.sm_scale = p.sm_scale;
  a.bias = to_bias(p.bias);
  return a;
}

bool same_dims(const ra_bwd_step_params& p, const ra_bwd_step_params& f) {
  return p.B == f.B && p.H == f.H && p.Lq == f.Lq && p.Lk == f.Lk && p.D == f.D && p.sm_scale == f.sm_scale;
}

bool same_strides(const ra_tensor& x, const ra_tensor& y) {
  return x.stride_b == y.stride_b && x.stride_h == y.stride_h && x.stride_l == y.stride_l;
}

// everything of a bias description that belongs to the launch or to the query shard
bool same_q_side(const ra_bias& x, const ra_bias& y) {
  return x.flags == y.flags && x.window == y.window && x.q_offset == y.q_offset &&
         x.q_segment_ids == y.q_segment_ids && x.q_segment_stride_b == y.q_segment_stride_b &&
         x.kv_segment_stride_b == y.kv_segment_stride_b && x.q_prefix == y.q_prefix &&
         x.q_prefix_stride_b == y.q_prefix_stride_b && x.kv_prefix_stride_b == y.kv_prefix_stride_b &&
         x.alibi_slopes == y.alibi_slopes && x.dense_stride_b == y.dense_stride_b &&
         x.dense_stride_h == y.dense_stride_h && x.dense_stride_q == y.dense_stride_q;
}

// ... and to the key/value shard
bool same_kv_side(const ra_bias& x, const ra_bias& y) {
  return x.flags == y.flags && x.window == y.window && x.kv_offset == y.kv_offset &&
         x.kv_segment_ids == y.kv_segment_ids && x.q_segment_stride_b == y.q_segment_stride_b &&
         x.kv_segment_stride_b == y.kv_segment_stride_b && x.kv_prefix == y.kv_prefix &&
         x.q_prefix_stride_b == y.q_prefix_stride_b && x.kv_prefix_stride_b == y.kv_prefix_stride_b &&
         x.alibi_slopes == y.alibi_slopes && x.dense_stride_b == y.dense_stride_b &&
         x.dense_stride_h == y.dense_stride_h && x.dense_stride_q == y.dense_stride_q;
}

// ---- launches that walk several shards, and several ring passes per launch ------------------------
// The travelling side of a step, as the shared table of a ring launch holds it.
struct KvEntry {
  const void* k; const void* v; int64_t off; const int32_t* seg; const int32_t* pre; const float* dense;
  bool operator==(const KvEntry& o) const {
    return k == o.k && v == o.v && off == o.off && seg == o.seg && pre == o.pre && dense == o.dense;
  }
};
struct QEntry {
  const void* q; const void* dout; const float* lse; const float* delta; int64_t off; const int32_t* seg;
  const int32_t* pre; const float* dense;
  bool operator==(const QEntry& o) const {
    return q == o.q && dout == o.dout && lse == o.lse && delta == o.delta && off == o.off && seg == o.seg &&
           pre == o.pre && dense == o.dense;
  }
};
KvEntry kv_entry(const ra_tensor& k, const ra_tensor& v, const ra_bias& b) {
  return KvEntry{k.ptr, v.ptr, b.kv_offset, b.kv_segment_ids, b.kv_prefix, b.dense_bias};
}
QEntry q_entry(const ra_bwd_step_params& p) {
  return QEntry{p.q.ptr, p.dout.ptr, p.lse, p.delta, p.bias.q_offset, p.bias.q_segment_ids, p.bias.q_prefix,
                p.bias.dense_bias};
}
void put(ra::KvShardList& t, int i, const KvEntry& e) {
  t.kv_off[i] = (int)e.off;
  t.k[i] = (const ra::bf16_t*)e.k;
  t.v[i] = (const ra::bf16_t*)e.v;
  t.kv_seg[i] = e.seg;
  t.kv_pre[i] = e.pre;
  t.dense[i] = e.dense;
}
void put(ra::QShardList& t, int i, const QEntry& e) {
  t.q_off[i] = (int)e.off;
  t.q[i] = (const ra::bf16_t*)e.q;
  t.dout[i] = (const ra::bf16_t*)e.dout;
  t.lse[i] = e.lse;
  t.delta[i] = e.delta;
  t.q_seg[i] = e.seg;
  t.q_pre[i] = e.pre;
  t.dense[i] = e.dense;
}

// Plans the launches of `n_passes` ring passes whose live steps (entries of the travelling side)
// are entries[first[p] .. first[p + 1]).  If every pass has at most kMaxShards live steps, there
// are at most kMaxPasses passes and the passes draw from at most kMaxShards distinct shards, ONE
// launch covers them all (heaviest pass first: it is dispatched first); otherwise every pass gets
// its own launches of at most kMaxShards steps each.  Ring is KvRing or QRing, `set_pass(ring,
// slot, p)` fills the resident side of pass p into slot `slot`, `launch(ring)` enqueues.
// `whole`: a whole-ring launch - passes without a live step take part too (their results are
// still to be written), and what does not fit one launch is refused (RA_ERR_TOO_LARGE, nothing
// launched): split into several launches a pass would need its intermediate state in memory.
template <typename Ring, typename Table, typename Entry, typename SetPass, typename Launch>
int run_passes(Table Ring::*table, const std::vector<Entry>& entries, const std::vector<int>& first, int n_passes,
               SetPass set_pass, Launch launch, bool whole = false) {
  std::vector<Entry> distinct;
  std::vector<int> index(entries.size());
  bool one_launch = n_passes <= ra::kMaxPasses;
  for (size_t i = 0; i < entries.size() && one_launch; ++i) {
    size_t j = 0;
    while (j < distinct.size() && !(distinct[j] == entries[i])) ++j;
    if (j == distinct.size()) {
      if ((int)distinct.size() == ra::kMaxShards) one_launch = false;
      else distinct.push_back(entries[i]);
    }
    index[i] = (int)j;
  }
  for (int p = 0; p < n_passes && one_launch; ++p) one_launch = first[p + 1] - first[p] <= ra::kMaxShards;
  Ring ring;
  memset(&ring, 0, sizeof(ring));
  if (one_launch) {
    for (size_t j = 0; j < distinct.size(); ++j) put(ring.*table, (int)j, distinct[j]);
    (ring.*table).n = (int)distinct.size();
    std::vector<int> by_weight;
    for (int p = 0; p < n_passes; ++p)
      if (whole || first[p + 1] > first[p]) by_weight.push_back(p);
    std::stable_sort(by_weight.begin(), by_weight.end(),
                     [&](int x, int y) { return first[x + 1] - first[x] > first[y + 1] - first[y]; });
    if (by_weight.empty()) return RA_OK;
    ring.n_pass = (int)by_weight.size();
    for (int slot = 0; slot < ring.n_pass; ++slot) {
      const int p = by_weight[slot];
      ring.count[slot] = (unsigned char)(first[p + 1] - first[p]);
      for (int i = first[p]; i < first[p + 1]; ++i) ring.order[slot][i - first[p]] = (unsigned char)index[i];
      set_pass(ring, slot, p);
    }
    return launch(ring);
  }
  if (whole)
    return fail(RA_ERR_TOO_LARGE, "a whole-ring launch takes at most %d passes that draw from at most %d distinct "
                                  "travelling shards; use the *_passes entry points", ra::kMaxPasses, ra::kMaxShards);
  for (int p = 0; p < n_passes; ++p) {
    for (int i0 = first[p]; i0 < first[p + 1]; i0 += ra::kMaxShards) {
      const int cnt = std::min(ra::kMaxShards, first[p + 1] - i0);
      memset(&ring, 0, sizeof(ring));
      for (int i = 0; i < cnt; ++i) {
        put(ring.*table, i, entries[i0 + i]);
        ring.order[0][i] = (unsigned char)i;
      }
      (ring.*table).n = cnt;
      ring.n_pass = 1;
      ring.count[0] = (unsigned char)cnt;
      set_pass(ring, 0, p);
      int rc = launch(ring);
      if (rc) return rc;
    }
  }
  return RA_OK;
}

// the fields of a bias description that every step of a launch must share
bool same_bias_shape(const ra_bias& x, const ra_bias& y) {
  return x.flags == y.flags && x.window == y.window && x.q_segment_stride_b == y.q_segment_stride_b &&
         x.kv_segment_stride_b == y.kv_segment_stride_b && x.q_prefix_stride_b == y.q_prefix_stride_b &&
         x.kv_prefix_stride_b == y.kv_prefix_stride_b && x.alibi_slopes == y.alibi_slopes &&
         x.dense_stride_b == y.dense_stride_b && x.dense_stride_h == y.dense_stride_h &&
         x.dense_stride_q == y.dense_stride_q;
}

// Where a whole-ring launch stores what it finished: pass p at `base + p * stride_pass` elements
// (second array for dV), element size `esize`, strides in elements.
struct RingResult {
  void* base;
  void* base2;
  float* lse;
  int dtype;  // RA_DTYPE_*
  int64_t stride_pass, stride_b, stride_h, stride_l;
};

int check_ring_result(const char* what, const RingResult& r) {
  if (!r.base) return fail(RA_ERR_NULL, "%s: NULL result pointer", what);
  if (r.dtype != RA_DTYPE_BF16 && r.dtype != RA_DTYPE_F32) return fail(RA_ERR_DTYPE, "unknown out_dtype %d", r.dtype);
  if ((r.stride_pass % 4) || (r.stride_b % 4) || (r.stride_h % 4) || (r.stride_l % 4))
    return fail(RA_ERR_ALIGN, "%s: result strides must be multiples of 4 elements", what);
  // the kernels store four elements at a time: 8 bytes of bf16 or 16 bytes of fp32
  const unsigned al = r.dtype == RA_DTYPE_F32 ? 16u : 8u;
  if (reinterpret_cast<uintptr_t>(r.base) % al || reinterpret_cast<uintptr_t>(r.base2) % al)
    return fail(RA_ERR_ALIGN, "%s: results must be aligned to four elements (%u bytes)", what, al);
  return RA_OK;
}

char* pass_slice(void* base, const RingResult& r, int p) {
  return (char*)base + (int64_t)p * r.stride_pass * (r.dtype == RA_DTYPE_F32 ? 4 : 2);
}

int check_pass_counts(const int32_t* steps_per_pass, int32_t n_passes, std::vector<int>& first) {
  if (n_passes < 0) return fail(RA_ERR_SHAPE, "n_passes is negative");
  if (n_passes > 0 && !steps_per_pass) return fail(RA_ERR_NULL, "steps_per_pass is NULL");
  first.assign(1, 0);
  for (int p = 0; p < n_passes; ++p) {
    if (steps_per_pass[p] < 0) return fail(RA_ERR_SHAPE, "steps_per_pass[%d] is negative", p);
    first.push_back(first.back() + steps_per_pass[p]);
  }
  return RA_OK;
}

int fwd_passes(const ra_fwd_step_params* steps, const std::vector<int>& first, int n_passes, void* stream,
               const RingResult* whole = nullptr) {
  const int total = first.back();
  if (total == 0) return RA_OK;
  if (!steps) return fail(RA_ERR_NULL, "steps is NULL");
  const ra_fwd_step_params& f = steps[0];
  for (int p = 0; p < n_passes; ++p) {
    for (int i = first[p]; i < first[p + 1]; ++i) {
      const ra_fwd_step_params& s = steps[i];
      const ra_fwd_step_params& h = steps[first[p]];  // head of the pass
      ra_fwd_step_params c = s;
      if (whole) c.o = c.m = c.l = reinterpret_cast<float*>(uintptr_t(16));  // not used: there is no carry
      int rc = ra_fwd_step_check(&c);
      if (rc) return rc;
      const bool shape = s.B == f.B && s.H == f.H && s.Lq == f.Lq && s.Lk == f.Lk && s.D == f.D &&
                         s.sm_scale == f.sm_scale && same_strides(s.q, f.q) && same_strides(s.k, f.k) &&
                         same_strides(s.v, f.v) && same_bias_shape(s.bias, f.bias);
      const bool pass = !memcmp(&s.q, &h.q, sizeof(ra_tensor)) &&
                        (whole || (s.o == h.o && s.m == h.m && s.l == h.l)) && same_q_side(s.bias, h.bias);
      if (!shape || !pass)
        return fail(RA_ERR_SHAPE, "steps[%d] differs from the first step of its pass in more than its key/value shard "
                                  "(k.ptr, v.ptr, kv_offset, kv_segment_ids, kv_prefix, dense_bias), or from "
                                  "steps[0] in shape, strides or bias terms", i);
    }
  }
  ra::FwdArgs a;
  a.q = to_arg(f.q);
  a.k = to_arg(f.k);
  a.v = to_arg(f.v);
  a.o = f.o;
  a.m = f.m;
  a.l = f.l;
  a.B = f.B;
  a.H = f.H;
  a.Lq = f.Lq;
  a.Lk = f.Lk;
  a.scale2 = f.sm_scale * kLog2eHost;
  a.bias = to_bias(f.bias);
  if (whole) {
    a.bias.flags |= whole->dtype == RA_DTYPE_F32 ? ra::kFlagWholeF32 : ra::kFlagWholeBf16;
    a.out_sb = whole->stride_b;  // in the slots of the carry pointers, which have no use here
    a.out_sh = whole->stride_h;
    a.out_sl = whole->stride_l;
  }
  // live steps only: a masked step is an identity on the carry
  std::vector<KvEntry> entries;
  std::vector<int> live_first(1, 0), head(n_passes, 0);
  for (int p = 0; p < n_passes; ++p) {
    head[p] = first[p];
    for (int i = first[p]; i < first[p + 1]; ++i)
      if (!ra_step_is_skippable(&steps[i].bias, steps[i].Lq, steps[i].Lk))
        entries.push_back(kv_entry(steps[i].k, steps[i].v, steps[i].bias));
    live_first.push_back((int)entries.size());
  }
  auto set_pass = [&](ra::KvRing& r, int slot, int p) {
    const ra_fwd_step_params& h = steps[head[p]];
    r.q_off[slot] = (int)h.bias.q_offset;
    r.q[slot] = (const ra::bf16_t*)h.q.ptr;
    r.x0[slot] = h.o;
    r.x1[slot] = h.m;
    r.x2[slot] = h.l;
    if (whole) {
      r.x0[slot] = reinterpret_cast<float*>(pass_slice(whole->base, *whole, p));
      r.x1[slot] = whole->lse + (int64_t)p * f.B * f.H * f.Lq;
      r.x2[slot] = nullptr;
    }
    r.q_seg[slot] = h.bias.q_segment_ids;
    r.q_pre[slot] = h.bias.q_prefix;
  };
  auto launch = [&](const ra::KvRing& r) -> int {
    hipError_t e = ra::launch_fwd_steps(a, r, f.D, kernel_mode(f.bias.flags), (hipStream_t)stream);
    return e == hipSuccess ? RA_OK : hip_fail(e, "forward ring launch");
  };
  return run_passes<ra::KvRing>(&ra::KvRing::kv, entries, live_first, n_passes, set_pass, launch, whole != nullptr);
}

int bwd_dq_passes(const ra_bwd_step_params* steps, const std::vector<int>& first, int n_passes, void* stream,
                  const RingResult* whole = nullptr) {
  const int total = first.back();
  if (total == 0) return RA_OK;
  if (!steps) return fail(RA_ERR_NULL, "steps is NULL");
  const ra_bwd_step_params& f = steps[0];
  for (int p = 0; p < n_passes; ++p) {
    for (int i = first[p]; i < first[p + 1]; ++i) {
      const ra_bwd_step_params& s = steps[i];
      const ra_bwd_step_params& h = steps[first[p]];
      ra_bwd_step_params c = s;
      if (whole) c.dq = c.dk = c.dv = reinterpret_cast<float*>(uintptr_t(16));  // not used: no accumulators
      int rc = ra_bwd_step_check(&c);
      if (rc) return rc;
      const bool shape = same_dims(s, f) && same_strides(s.q, f.q) && same_strides(s.dout, f.dout) &&
                         same_strides(s.k, f.k) && same_strides(s.v, f.v) && same_bias_shape(s.bias, f.bias);
      const bool pass = !memcmp(&s.q, &h.q, sizeof(ra_tensor)) && !memcmp(&s.dout, &h.dout, sizeof(ra_tensor)) &&
                        s.lse == h.lse && s.delta == h.delta && (whole || s.dq == h.dq) && same_q_side(s.bias, h.bias);
      if (!shape || !pass)
        return fail(RA_ERR_SHAPE, "steps[%d] differs from the first step of its pass in more than its key/value shard "
                                  "(k.ptr, v.ptr, dk, dv, kv_offset, kv_segment_ids, kv_prefix, dense_bias), or from "
                                  "steps[0] in shape, strides or bias terms", i);
    }
  }
  ra::BwdArgs a = to_bwd_args(f);
  if (whole) {
    a.bias.flags |= ra::kFlagWholeBf16;
    a.out_sb = whole->stride_b;  // in the slots of the accumulator pointers, which have no use here
    a.out_sh = whole->stride_h;
    a.out_sl = whole->stride_l;
  }
  std::vector<KvEntry> entries;
  std::vector<int> live_first(1, 0);
  for (int p = 0; p < n_passes; ++p) {
    for (int i = first[p]; i < first[p + 1]; ++i)
      if (!ra_step_is_skippable(&steps[i].bias, steps[i].Lq, steps[i].Lk))  // contributes nothing
        entries.push_back(kv_entry(steps[i].k, steps[i].v, steps[i].bias));
    live_first.push_back((int)entries.size());
  }
  auto set_pass = [&](ra::KvRing& r, int slot, int p) {
    const ra_bwd_step_params& h = steps[first[p]];
    r.q_off[slot] = (int)h.bias.q_offset;
    r.q[slot] = (const ra::bf16_t*)h.q.ptr;
    r.dout[slot] = (const ra::bf16_t*)h.dout.ptr;
    r.x0[slot] = whole ? reinterpret_cast<float*>(pass_slice(whole->base, *whole, p)) : h.dq;
    r.x1[slot] = const_cast<float*>(h.lse);
    r.x2[slot] = const_cast<float*>(h.delta);
    r.q_seg[slot] = h.bias.q_segment_ids;
    r.q_pre[slot] = h.bias.q_prefix;
  };
  auto launch = [&](const ra::KvRing& r) -> int {
    hipError_t e = ra::launch_bwd_dq_steps(a, r, f.D, kernel_mode(f.bias.flags), (hipStream_t)stream);
    return e == hipSuccess ? RA_OK : hip_fail(e, "dQ ring launch");
  };
  return run_passes<ra::KvRing>(&ra::KvRing::kv, entries, live_first, n_passes, set_pass, launch, whole != nullptr);
}

int bwd_dkdv_passes(const ra_bwd_step_params* steps, const std::vector<int>& first, int n_passes, void* stream,
                    const RingResult* whole = nullptr) {
  const int total = first.back();
  if (total == 0) return RA_OK;
  if (!steps) return fail(RA_ERR_NULL, "steps is NULL");
  const ra_bwd_step_params& f = steps[0];
  for (int p = 0; p < n_passes; ++p) {
    for (int i = first[p]; i < first[p + 1]; ++i) {
      const ra_bwd_step_params& s = steps[i];
      const ra_bwd_step_params& h = steps[first[p]];
      ra_bwd_step_params c = s;
      if (whole) c.dq = c.dk = c.dv = reinterpret_cast<float*>(uintptr_t(16));  // not used: no accumulators
      int rc = ra_bwd_step_check(&c);
      if (rc) return rc;
      const bool shape = same_dims(s, f) && same_strides(s.q, f.q) && same_strides(s.dout, f.dout) &&
                         same_strides(s.k, f.k) && same_strides(s.v, f.v) && same_bias_shape(s.bias, f.bias);
      const bool pass = !memcmp(&s.k, &h.k, sizeof(ra_tensor)) && !memcmp(&s.v, &h.v, sizeof(ra_tensor)) &&
                        (whole || (s.dk == h.dk && s.dv == h.dv)) && same_kv_side(s.bias, h.bias);
      if (!shape || !pass)
        return fail(RA_ERR_SHAPE, "steps[%d] differs from the first step of its pass in more than its query shard (q.ptr, "
                                  "dout.ptr, lse, delta, dq, q_offset, q_segment_ids, q_prefix, dense_bias), or from "
                                  "steps[0] in shape, strides or bias terms", i);
    }
  }
  ra::BwdArgs a = to_bwd_args(f);
  if (whole) {
    a.bias.flags |= ra::kFlagWholeBf16;
    a.out_sb = whole->stride_b;  // in the slots of the accumulator pointers, which have no use here
    a.out_sh = whole->stride_h;
    a.out_sl = whole->stride_l;
  }
  std::vector<QEntry> entries;
  std::vector<int> live_first(1, 0);
  for (int p = 0; p < n_passes; ++p) {
    for (int i = first[p]; i < first[p + 1]; ++i)
      if (!ra_step_is_skippable(&steps[i].bias, steps[i].Lq, steps[i].Lk))  // contributes nothing
        entries.push_back(q_entry(steps[i]));
    live_first.push_back((int)entries.size());
  }
  auto set_pass = [&](ra::QRing& r, int slot, int p) {
    const ra_bwd_step_params& h = steps[first[p]];
    r.kv_off[slot] = (int)h.bias.kv_offset;
    r.k[slot] = (const ra::bf16_t*)h.k.ptr;
    r.v[slot] = (const ra::bf16_t*)h.v.ptr;
    r.dk[slot] = whole ? reinterpret_cast<float*>(pass_slice(whole->base, *whole, p)) : h.dk;
    r.dv[slot] = whole ? reinterpret_cast<float*>(pass_slice(whole->base2, *whole, p)) : h.dv;
    r.kv_seg[slot] = h.bias.kv_segment_ids;
    r.kv_pre[slot] = h.bias.kv_prefix;
  };
  auto launch = [&](const ra::QRing& r) -> int {
    hipError_t e = ra::launch_bwd_dkdv_steps(a, r, f.D, kernel_mode(f.bias.flags), (hipStream_t)stream);
    return e == hipSuccess ? RA_OK : hip_fail(e, "dK/dV ring launch");
  };
  return run_passes<ra::QRing>(&ra::QRing::q, entries, live_first, n_passes, set_pass, launch, whole != nullptr);
}

}  // namespace

extern "C" {

int ra_version(void) { return 1006; }

const char* ra_last_error(void) { return g_err; }

int ra_step_is_skippable(const ra_bias* bias, int32_t Lq, int32_t Lk) {
  if (!bias || Lq <= 0 || Lk <= 0) return 0;
  if (bias->flags & RA_BIAS_PREFIX) return 0;
  const int64_t qlo = bias->q_offset, qhi = bias->q_offset + Lq - 1;
  const int64_t klo = bias->kv_offset, khi = bias->kv_offset + Lk - 1;
  if ((bias->flags & RA_BIAS_CAUSAL) && klo > qhi) return 1;
  if (bias->flags & RA_BIAS_WINDOW) {
    if (qlo - khi >= bias->window) return 1;
    if (!(bias->flags & RA_BIAS_CAUSAL) && klo - qhi >= bias->window) return 1;
  }
  return 0;
}

int ra_fwd_step_check(const ra_fwd_step_params* p) {
  if (!p) return fail(RA_ERR_NULL, "params is NULL");
  int rc = check_dims(p->B, p->H, p->Lq, p->Lk, p->D);
  if (rc) return rc;
  if ((rc = check_tensor("q", p->q, p->D))) return rc;
  if ((rc = check_tensor("k", p->k, p->D))) return rc;
  if ((rc = check_tensor("v", p->v, p->D))) return rc;
  if (!p->o || !p->m || !p->l) return fail(RA_ERR_NULL, "carry pointer (o, m or l) is NULL");
  if (!aligned16(p->o)) return fail(RA_ERR_ALIGN, "o is not 16-byte aligned");
  if (!(p->sm_scale > 0.f) || p->sm_scale > 3.0e38f)
    return fail(RA_ERR_SHAPE, "sm_scale must be a positive finite number");
  return check_bias(p->bias, p->Lq, p->Lk);
}

int ra_bwd_step_check(const ra_bwd_step_params* p) {
  if (!p) return fail(RA_ERR_NULL, "params is NULL");
  int rc = check_dims(p->B, p->H, p->Lq, p->Lk, p->D);
  if (rc) return rc;
  if ((rc = check_tensor("q", p->q, p->D))) return rc;
  if ((rc = check_tensor("k", p->k, p->D))) return rc;
  if ((rc = check_tensor("v", p->v, p->D))) return rc;
  if ((rc = check_tensor("dout", p->dout, p->D))) return rc;
  if (!p->lse || !p->delta) return fail(RA_ERR_NULL, "lse or delta is NULL");
  if (!p->dq || !p->dk || !p->dv) return fail(RA_ERR_NULL, "gradient accumulator (dq, dk or dv) is NULL");
  if (!aligned16(p->dq) || !aligned16(p->dk) || !aligned16(p->dv))
    return fail(RA_ERR_ALIGN, "gradient accumulators must be 16-byte aligned");
  if (!(p->sm_scale > 0.f) || p->sm_scale > 3.0e38f)
    return fail(RA_ERR_SHAPE, "sm_scale must be a positive finite number");
  return check_bias(p->bias, p->Lq, p->Lk);
}

int ra_fwd_init(float* o, float* m, float* l, int32_t B, int32_t H, int32_t Lq, int32_t D, void* stream) {
  if (!o || !m || !l) return fail(RA_ERR_NULL, "carry pointer (o, m or l) is NULL");
  int rc = check_dims(B, H, Lq, 1, D);
  if (rc) return rc;
  hipError_t e = ra::launch_fwd_init(o, m, l, (long long)B * H * Lq, D, (hipStream_t)stream);
  return e == hipSuccess ? RA_OK : hip_fail(e, "ra_fwd_init launch");
}

int64_t ra_dense_map_bytes(int64_t stride_b, int64_t stride_h, int32_t B, int32_t H, int32_t Lq, int32_t Lk) {
  if (B <= 0 || H <= 0 || Lq <= 0 || Lk <= 0) return 0;
  const int64_t cells = (int64_t)((Lq + 31) / 32) * ((Lk + 31) / 32);
  return (stride_b ? B : 1) * (int64_t)(stride_h ? H : 1) * cells;
}

int ra_dense_map(const float* dense_bias, int64_t stride_b, int64_t stride_h, int64_t stride_q, int32_t B,
                 int32_t H, int32_t Lq, int32_t Lk, uint8_t* map, void* stream) {
  if (!dense_bias || !map) return fail(RA_ERR_NULL, "ra_dense_map: NULL pointer");
  if (B <= 0 || H <= 0 || Lq <= 0 || Lk <= 0)
    return fail(RA_ERR_SHAPE, "ra_dense_map: bad shape B=%d H=%d Lq=%d Lk=%d", B, H, Lq, Lk);
  if (Lq > kMaxSegLen || Lk > kMaxSegLen)
    return fail(RA_ERR_SHAPE, "ra_dense_map: shards of at most %d tokens", kMaxSegLen);
  if (((uintptr_t)dense_bias & 3) != 0) return fail(RA_ERR_ALIGN, "dense_bias is not 4-byte aligned");
  if (stride_q < Lk || stride_b < 0 || stride_h < 0)
    return fail(RA_ERR_BIAS, "dense bias strides: stride_q must be at least Lk, stride_b / stride_h "
                             "non-negative (0 broadcasts)");
  const int nb = stride_b ? B : 1, nh = stride_h ? H : 1;
  if ((int64_t)nb * nh > 65535) return fail(RA_ERR_SHAPE, "ra_dense_map: more than 65535 (batch, head) blocks");
  hipError_t e = ra::launch_dense_map(dense_bias, stride_b, stride_h, stride_q, nb, nh, Lq, Lk, map,
                                      (hipStream_t)stream);
  return e == hipSuccess ? RA_OK : hip_fail(e, "ra_dense_map launch");
}

int ra_fwd_step(const ra_fwd_step_params* p, void* stream) {
  int rc = ra_fwd_step_check(p);
  if (rc) return rc;
  if (ra_step_is_skippable(&p->bias, p->Lq, p->Lk)) return RA_OK;  // identity on the carry
  ra::FwdArgs a;
  a.q = to_arg(p->q);
  a.k = to_arg(p->k);
  a.v = to_arg(p->v);
  a.o = p->o;
  a.m = p->m;
  a.l = p->l;
  a.B = p->B;
  a.H = p->H;
  a.Lq = p->Lq;
  a.Lk = p->Lk;
  a.scale2 = p->sm_scale * kLog2eHost;
  a.bias = to_bias(p->bias);
  hipError_t e = ra::launch_fwd_step(a, p->D, kernel_mode(p->bias.flags), (hipStream_t)stream);
  return e == hipSuccess ? RA_OK : hip_fail(e, "ra_fwd_step launch");
}

int ra_fwd_steps(const ra_fwd_step_params* steps, int32_t n_steps, void* stream) {
  if (n_steps < 0) return fail(RA_ERR_SHAPE, "n_steps is negative");
  return fwd_passes(steps, std::vector<int>{0, n_steps}, 1, stream);
}

int ra_fwd_passes(const ra_fwd_step_params* steps, const int32_t* steps_per_pass, int32_t n_passes, void* stream) {
  std::vector<int> first;
  int rc = check_pass_counts(steps_per_pass, n_passes, first);
  return rc ? rc : fwd_passes(steps, first, n_passes, stream);
}

int ra_fwd_finalize_passes(const float* o, const float* m, const float* l, void* out, int32_t out_dtype,
                           int64_t out_stride_pass, int64_t out_stride_b, int64_t out_stride_h,
                           int64_t out_stride_l, float* lse, int32_t n_passes, int32_t B, int32_t H, int32_t Lq,
                           int32_t D, void* stream) {
  if (!o || !m || !l || !out || !lse) return fail(RA_ERR_NULL, "ra_fwd_finalize: NULL pointer");
  if (n_passes <= 0 || n_passes > (1 << 16)) return fail(RA_ERR_SHAPE, "n_passes must lie in [1, 65536]");
  int rc = check_dims(B, H, Lq, 1, D);
  if (rc) return rc;
  if ((int64_t)n_passes * B * H > (1 << 20)) return fail(RA_ERR_SHAPE, "n_passes*B*H too large");
  if (out_dtype != RA_DTYPE_BF16 && out_dtype != RA_DTYPE_F32)
    return fail(RA_ERR_DTYPE, "unknown out_dtype %d", out_dtype);
  if ((out_stride_pass % 4) || (out_stride_b % 4) || (out_stride_h % 4) || (out_stride_l % 4))
    return fail(RA_ERR_ALIGN, "out strides must be multiples of 4 elements");
  // the kernel stores four elements at a time: 8 bytes of bf16 or 16 bytes of fp32
  if (reinterpret_cast<uintptr_t>(out) % (out_dtype == RA_DTYPE_F32 ? 16u : 8u))
    return fail(RA_ERR_ALIGN, "out must be aligned to four elements (%d bytes)", out_dtype == RA_DTYPE_F32 ? 16 : 8);
  if (!aligned16(o)) return fail(RA_ERR_ALIGN, "o is not 16-byte aligned");
  hipError_t e = ra::launch_fwd_finalize(o, m, l, out, out_dtype == RA_DTYPE_F32, out_stride_pass, out_stride_b,
                                         out_stride_h, out_stride_l, lse, n_passes, B, H, Lq, D,
                                         (hipStream_t)stream);
  return e == hipSuccess ? RA_OK : hip_fail(e, "ra_fwd_finalize launch");
}

int ra_fwd_finalize(const float* o, const float* m, const float* l, void* out, int32_t out_dtype,
                    int64_t out_stride_b, int64_t out_stride_h, int64_t out_stride_l, float* lse,
                    int32_t B, int32_t H, int32_t Lq, int32_t D, void* stream) {
  return ra_fwd_finalize_passes(o, m, l, out, out_dtype, 0, out_stride_b, out_stride_h, out_stride_l, lse, 1, B, H,
                                Lq, D, stream);
}

int ra_bwd_delta_passes(const void* out, int32_t out_dtype, int64_t out_stride_pass, int64_t out_stride_b,
                        int64_t out_stride_h, int64_t out_stride_l, const ra_tensor* dout,
                        int64_t dout_stride_pass, float* delta, int32_t n_passes, int32_t B, int32_t H,
                        int32_t Lq, int32_t D, void* stream) {
  if (!out || !dout || !delta) return fail(RA_ERR_NULL, "ra_bwd_delta: NULL pointer");
  if (n_passes <= 0 || n_passes > (1 << 16)) return fail(RA_ERR_SHAPE, "n_passes must lie in [1, 65536]");
  int rc = check_dims(B, H, Lq, 1, D);
  if (rc) return rc;
  if ((int64_t)n_passes * B * H > (1 << 20)) return fail(RA_ERR_SHAPE, "n_passes*B*H too large");
  if ((rc = check_tensor("dout", *dout, D))) return rc;
  if (out_dtype != RA_DTYPE_BF16 && out_dtype != RA_DTYPE_F32)
    return fail(RA_ERR_DTYPE, "unknown out_dtype %d", out_dtype);
  if (!aligned16(out) || (out_stride_pass % 8) || (out_stride_b % 8) || (out_stride_h % 8) || (out_stride_l % 8) ||
      (dout_stride_pass % 8))
    return fail(RA_ERR_ALIGN, "out must be 16-byte aligned with strides that are multiples of 8");
  hipError_t e = ra::launch_bwd_delta(out, out_dtype == RA_DTYPE_F32, out_stride_pass, out_stride_b, out_stride_h,
                                      out_stride_l, to_arg(*dout), dout_stride_pass, delta, n_passes, B, H, Lq, D,
                                      (hipStream_t)stream);
  return e == hipSuccess ? RA_OK : hip_fail(e, "ra_bwd_delta launch");
}

int ra_bwd_delta(const void* out, int32_t out_dtype, int64_t out_stride_b, int64_t out_stride_h,
                 int64_t out_stride_l, const ra_tensor* dout, float* delta, int32_t B, int32_t H,
                 int32_t Lq, int32_t D, void* stream) {
  return ra_bwd_delta_passes(out, out_dtype, 0, out_stride_b, out_stride_h, out_stride_l, dout, 0, delta, 1, B, H, Lq,
                             D, stream);
}

int ra_bwd_step(const ra_bwd_step_params* p, void* stream) { return ra_bwd_step_parts(p, 3, stream); }

int ra_bwd_step_parts(const ra_bwd_step_params* p, int32_t parts, void* stream) {
  int rc = ra_bwd_step_check(p);
  if (rc) return rc;
  if (parts < 1 || parts > 3) return fail(RA_ERR_SHAPE, "parts must be 1, 2 or 3 (got %d)", parts);
  if (ra_step_is_skippable(&p->bias, p->Lq, p->Lk)) return RA_OK;  // contributes nothing
  const ra::BwdArgs a = to_bwd_args(*p);
  hipError_t e = ra::launch_bwd_step(a, p->D, kernel_mode(p->bias.flags), parts, (hipStream_t)stream);
  return e == hipSuccess ? RA_OK : hip_fail(e, "ra_bwd_step launch");
}

int ra_bwd_dq_steps(const ra_bwd_step_params* steps, int32_t n_steps, void* stream) {
  if (n_steps < 0) return fail(RA_ERR_SHAPE, "n_steps is negative");
  return bwd_dq_passes(steps, std::vector<int>{0, n_steps}, 1, stream);
}

int ra_bwd_dkdv_steps(const ra_bwd_step_params* steps, int32_t n_steps, void* stream) {
  if (n_steps < 0) return fail(RA_ERR_SHAPE, "n_steps is negative");
  return bwd_dkdv_passes(steps, std::vector<int>{0, n_steps}, 1, stream);
}

int ra_bwd_dq_passes(const ra_bwd_step_params* steps, const int32_t* steps_per_pass, int32_t n_passes,
                     void* stream) {
  std::vector<int> first;
  int rc = check_pass_counts(steps_per_pass, n_passes, first);
  return rc ? rc : bwd_dq_passes(steps, first, n_passes, stream);
}

int ra_bwd_dkdv_passes(const ra_bwd_step_params* steps, const int32_t* steps_per_pass, int32_t n_passes,
                       void* stream) {
  std::vector<int> first;
  int rc = check_pass_counts(steps_per_pass, n_passes, first);
  return rc ? rc : bwd_dkdv_passes(steps, first, n_passes, stream);
}

// every pass of a whole-ring launch needs a head block to take its resident side from
static int check_whole(const std::vector<int>& first, int n_passes) {
  for (int p = 0; p < n_passes; ++p)
    if (first[p + 1] == first[p]) return fail(RA_ERR_SHAPE, "pass %d has no block", p);
  return RA_OK;
}

int ra_fwd_ring(const ra_fwd_step_params* steps, const int32_t* steps_per_pass, int32_t n_passes, void* out,
                int32_t out_dtype, int64_t out_stride_pass, int64_t out_stride_b, int64_t out_stride_h,
                int64_t out_stride_l, float* lse, void* stream) {
  std::vector<int> first;
  int rc = check_pass_counts(steps_per_pass, n_passes, first);
  if (rc || (rc = check_whole(first, n_passes))) return rc;
  if (!lse) return fail(RA_ERR_NULL, "ra_fwd_ring: lse is NULL");
  const RingResult r{out, nullptr, lse, out_dtype, out_stride_pass, out_stride_b, out_stride_h, out_stride_l};
  if ((rc = check_ring_result("ra_fwd_ring", r))) return rc;
  return fwd_passes(steps, first, n_passes, stream, &r);
}

int ra_bwd_dq_ring(const ra_bwd_step_params* steps, const int32_t* steps_per_pass, int32_t n_passes, void* dq,
                   int64_t stride_pass, int64_t stride_b, int64_t stride_h, int64_t stride_l, void* stream) {
  std::vector<int> first;
  int rc = check_pass_counts(steps_per_pass, n_passes, first);
  if (rc || (rc = check_whole(first, n_passes))) return rc;
  const RingResult r{dq, nullptr, nullptr, RA_DTYPE_BF16, stride_pass, stride_b, stride_h, stride_l};
  if ((rc = check_ring_result("ra_bwd_dq_ring", r))) return rc;
  return bwd_dq_passes(steps, first, n_passes, stream, &r);
}

int ra_bwd_dkdv_ring(const ra_bwd_step_params* steps, const int32_t* steps_per_pass, int32_t n_passes, void* dk,
                     void* dv, int64_t stride_pass, int64_t stride_b, int64_t stride_h, int64_t stride_l,
                     void* stream) {
  std::vector<int> first;
  int rc = check_pass_counts(steps_per_pass, n_passes, first);
  if (rc || (rc = check_whole(first, n_passes))) return rc;
  if (!dv) return fail(RA_ERR_NULL, "ra_bwd_dkdv_ring: dv is NULL");
  const RingResult r{dk, dv, nullptr, RA_DTYPE_BF16, stride_pass, stride_b, stride_h, stride_l};
  if ((rc = check_ring_result("ra_bwd_dkdv_ring", r))) return rc;
  return bwd_dkdv_passes(steps, first, n_passes, stream, &r);
}

int ra_bwd_finalize_passes(const float* acc, void* out, int64_t out_stride_pass, int64_t out_stride_b,
                           int64_t out_stride_h, int64_t out_stride_l, int32_t n_passes, int32_t B, int32_t H,
                           int32_t L, int32_t D, void* stream) {
  if (!acc || !out) return fail(RA_ERR_NULL, "ra_bwd_finalize: NULL pointer");
  if (n_passes <= 0 || n_passes > (1 << 16)) return fail(RA_ERR_SHAPE, "n_passes must lie in [1, 65536]");
  int rc = check_dims(B, H, L, 1, D);
  if (rc) return rc;
  if ((int64_t)n_passes * B * H > (1 << 20)) return fail(RA_ERR_SHAPE, "n_passes*B*H too large");
  if ((out_stride_pass % 4) || (out_stride_b % 4) || (out_stride_h % 4) || (out_stride_l % 4))
    return fail(RA_ERR_ALIGN, "out strides must be multiples of 4 elements");
  // the kernel loads 16 bytes of fp32 and stores 8 bytes of bf16 at a time
  if (reinterpret_cast<uintptr_t>(out) % 8u) return fail(RA_ERR_ALIGN, "out must be 8-byte aligned");
  if (!aligned16(acc)) return fail(RA_ERR_ALIGN, "acc is not 16-byte aligned");
  hipError_t e = ra::launch_bwd_finalize(acc, out, out_stride_pass, out_stride_b, out_stride_h, out_stride_l,
                                         n_passes, B, H, L, D, (hipStream_t)stream);
  return e == hipSuccess ? RA_OK : hip_fail(e, "ra_bwd_finalize launch");
}

int ra_bwd_finalize(const float* acc, void* out, int64_t out_stride_b, int64_t out_stride_h,
                    int64_t out_stride_l, int32_t B, int32_t H, int32_t L, int32_t D, void* stream) {
  return ra_bwd_finalize_passes(acc, out, 0, out_stride_b, out_stride_h, out_stride_l, 1, B, H, L, D, stream);
}

}  // extern "C"
