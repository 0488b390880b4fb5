// The schedules of the collectives over simulated ranks: which slices the last
// rank to post launches for an all-reduce, reduce, reduce-scatter, all-gather,
// all-to-all(v), gather, scatter, broadcast and the custom all-reduce hook.
//
// Reference behaviour followed:
//   chunk/slice/red-slice  flagcx/runner/uni_runner_impl.cc:661-1007 (sliced ring
//                          all-reduce), :1009-1264 (ring reduce-scatter),
//                          :1266-1557 (tree reduce)
//   host-path schedule ... flagcx/service/bootstrap.cc:787-942,1039-1066
//   nranks == 1 .......... copy if out of place, else nothing (:669-691)
//   alltoallv addressing . flagcx/service/bootstrap.cc:1253-1279
//   custom allreduce ..... flagcx/adaptor/kernel/nvidia/custom_allreduce.cu:604-677
// The transport between ranks is elided: a rank reads its peer's buffer where
// the reference would receive a copy of it.
#include "fx_sim_internal.hpp"

namespace fxsim {


// More inputs than a slice descriptor carries: such pieces go through the
// runtime-k kernel, one launch each, so pieces that continue each other in the
// send buffers and in the output are gathered into one run first (the
// red-slice split alone cuts a 64 MiB all-reduce over 16 ranks into 512 pieces
// of 128 KiB).
struct KwayRun {
  size_t sendOff = 0, cnt = 0;
  void *out = nullptr;
  int first = 0;
};

flagcxResult_t launchRun(const Ctx &c, KwayRun &run) {
  if (run.cnt == 0) return flagcxSuccess;
  PtrList in;
  in.resize((size_t)c.n);
  for (int j = 0; j < c.n; j++) in[j] = cadd(c.send(j), run.sendOff * c.ts);
  const flagcxResult_t rc = R(fx_reduce_copy(run.out, in.data(), c.n, run.cnt, c.g->dtype, c.g->op, run.first, c.s));
  run = KwayRun();
  return rc;
}

// k-way reduce of element range [off, off+cnt) of every rank's sendbuff (+sendBase
// elements) into out, in order first, first+1, ...
flagcxResult_t kway(const Ctx &c, SliceList &descs, KwayRun &run, size_t sendOff, size_t cnt, void *out, int first) {
  if (cnt == 0) return flagcxSuccess;
  if (c.n <= FX_MAX_SLICE_INPUTS) {
    fxSliceDesc d;
    memset(&d, 0, sizeof(d));
    for (int j = 0; j < c.n; j++) d.in[j] = cadd(c.send(mod(first + j, c.n)), sendOff * c.ts);
    d.out = out;
    d.count = cnt;
    descs.push_back(d);
    return flagcxSuccess;
  }
  if (run.cnt && first == run.first && sendOff == run.sendOff + run.cnt && out == madd(run.out, run.cnt * c.ts)) {
    run.cnt += cnt;
    return flagcxSuccess;
  }
  const flagcxResult_t rc = launchRun(c, run);
  run.sendOff = sendOff;
  run.cnt = cnt;
  run.out = out;
  run.first = first;
  return rc;
}

flagcxResult_t flushKway(const Ctx &c, SliceList &descs, KwayRun &run) {
  flagcxResult_t rc = launchRun(c, run);
  if (rc != flagcxSuccess || descs.empty()) return rc;
  rc = R(fx_reduce_slices(descs.data(), descs.size(), c.n, c.g->dtype, c.g->op, c.s));
  descs.clear();
  return rc;
}

// The many-rank kernels store one result to several buffers with shared byte
// offsets: the receive buffers must agree in their low four address bits.
inline bool recvsAlignedAlike(const Ctx &c) {
  for (int r = 1; r < c.n; r++)
    if ((((uintptr_t)c.recv(r) ^ (uintptr_t)c.recv(0)) & 15u) != 0) return false;
  return true;
}

// One read, n stores: usable when both the inputs and the outputs of a
// descriptor fit its eight slots.
inline bool canBroadcast(const Ctx &c) { return c.n <= FX_MAX_SLICE_INPUTS; }

// Visit the (slice, red-slice) pieces of a chunk of ccnt elements at element
// offset coff, exactly as the reference nests its three splits.
template <class F>
flagcxResult_t forPieces(const Group *g, size_t ccnt, size_t coff, size_t nred, F f) {
  for (size_t s = 0; s < (size_t)g->nslices; s++) {
    size_t scnt, soff;
    fx_split(ccnt, (size_t)g->nslices, s, &scnt, &soff);
    for (size_t q = 0; q < nred; q++) {
      size_t rcnt, roff;
      fx_split(scnt, nred, q, &rcnt, &roff);
      flagcxResult_t rc = f(coff + soff + roff, soff + roff, rcnt);
      if (rc != flagcxSuccess) return rc;
    }
  }
  return flagcxSuccess;
}

// ---- the host path's schedule (FX_ORDER_HOST) ----
// Element range of chunk i: ceil(size / n) bytes rounded up to whole elements,
// the last non-empty chunk short, later ones empty (bootstrap.cc:900-922).
void hostChunk(size_t count, int n, int i, size_t *cnt, size_t *off) {
  const size_t chunk = (count + (size_t)n - 1) / (size_t)n;  // same as the byte formula divided by the element size
  if (chunk * (size_t)i >= count) {
    *off = count;
    *cnt = 0;
  } else {
    *off = chunk * (size_t)i;
    *cnt = (chunk * (size_t)(i + 1) >= count) ? count - *off : chunk;
  }
}

// Rank order in which a left-to-right fold reproduces the host ring's result for
// chunk c.  The ring computes x_c (op) (x_{c-1} (op) (.. (x_{c+2} (op) x_{c+1}))),
// local operand first (bootstrap.cc:805-871).  For sum / prod / avg the operands
// of one step commute bit for bit, so the fold runs c+1, c+2, .., c.  For max /
// min of integers ((a < b) ? b : a keeps the LOCAL value on a tie) the fold keeps
// its accumulator on a tie instead, so it runs c, c-1, .., c+1: either way the
// last rank of the ring wins ties.  (Floating max / min do not come here: NaN
// makes them order-dependent in a way only the step-by-step chain reproduces.)
void hostOrder(int c, int n, int op, std::vector<int> &order) {
  order.resize(n);
  const bool select = (op == flagcxMax || op == flagcxMin);
  for (int j = 0; j < n; j++) order[j] = select ? mod(c - j, n) : mod(c + 1 + j, n);
}

// Host-order reduce of `nchunks` element ranges (chunk i = [off[i], off[i]+cnt[i]) of
// every send buffer, folded in hostOrder(chunkId[i])) into outs[i][0..nout-1].
struct HostPiece {
  int chunk;
  size_t off, cnt;
  std::vector<void *> outs;
};

// max / min of floating types, exactly as the host ring evaluates them: n-1
// two-input steps res = local (op) received (bootstrap.cc:853-871), the local
// operand first, so that a NaN met on the way decides the result the way it
// does there (std::max / std::min return their FIRST argument whenever the
// comparison is false).  A left-to-right k-way fold cannot express that: once
// rank j's NaN has been kept by rank j, everything folded before it is lost.
// Step j of chunk c: local rank c+1+j, received = the previous partial (rank
// c+1's data in step 1).  Partials travel through scratch; the last step, whose
// local rank is c itself, writes the outputs.  One launch per step for all chunks.
flagcxResult_t chainHostPieces(const Ctx &c, const std::vector<HostPiece> &pieces) {
  Group *g = c.g;
  const int n = c.n;
  // Up to eight ranks: the whole chain of a piece in registers, one launch for
  // all pieces, every input read once (in[0] = rank c+1's data, in[j] = the
  // local operand of step j).  Outputs that do not share their offset within 16
  // bytes fall through to the step-by-step form below.
  if (n <= FX_MAX_SLICE_INPUTS) {
    BcastList bd;
    bool alike = true;
    int nout = 1;
    for (const HostPiece &p : pieces) {
      if (p.cnt == 0) continue;
      nout = (int)p.outs.size();
      if (nout > FX_MAX_SLICE_INPUTS) alike = false;
      fxBcastDesc d;
      memset(&d, 0, sizeof(d));
      for (int j = 0; j < n; j++) d.in[j] = cadd(c.send(mod(p.chunk + 1 + j, n)), p.off * c.ts);
      for (int o = 0; o < nout && o < FX_MAX_SLICE_INPUTS; o++) {
        d.out[o] = p.outs[o];
        alike = alike && ((((uintptr_t)p.outs[o] ^ (uintptr_t)p.outs[0]) & 15u) == 0);
      }
      d.count = p.cnt;
      bd.push_back(d);
    }
    if (bd.empty()) return flagcxSuccess;
    if (alike) return R(fx_reduce_ordered(bd.data(), bd.size(), n, nout, g->dtype, g->op, FX_FOLD_KEEP_LOCAL, c.s));
  }
  std::vector<size_t> soff(pieces.size(), 0);
  size_t total = 0;
  for (size_t i = 0; i < pieces.size(); i++) {
    soff[i] = total;
    total += (pieces[i].cnt * c.ts + 255) & ~(size_t)255;
  }
  if (total == 0) return flagcxSuccess;
  if (n > 2) {
    flagcxResult_t rc = ensureScratch(g, total, c.s);
    if (rc != flagcxSuccess) return rc;
  }
  SliceList plain, copies;
  BcastList bcast;
  int nout = 1;
  for (int j = 1; j < n; j++) {
    plain.clear();
    for (size_t i = 0; i < pieces.size(); i++) {
      const HostPiece &p = pieces[i];
      if (p.cnt == 0) continue;
      const void *local = cadd(c.send(mod(p.chunk + 1 + j, n)), p.off * c.ts);
      const void *received = (j == 1) ? cadd(c.send(mod(p.chunk + 1, n)), p.off * c.ts)
                                      : (const void *)madd(g->scratch, soff[i]);
      nout = (int)p.outs.size();
      if (j == n - 1 && nout > 1 && nout <= FX_MAX_SLICE_INPUTS) {
        fxBcastDesc d;
        memset(&d, 0, sizeof(d));
        d.in[0] = local;
        d.in[1] = received;
        for (int o = 0; o < nout; o++) d.out[o] = p.outs[o];
        d.count = p.cnt;
        bcast.push_back(d);
        continue;
      }
      fxSliceDesc d;
      memset(&d, 0, sizeof(d));
      d.in[0] = local;
      d.in[1] = received;
      d.out = (j == n - 1) ? p.outs[0] : madd(g->scratch, soff[i]);
      d.count = p.cnt;
      plain.push_back(d);
      if (j == n - 1)
        for (int o = 1; o < nout; o++) copies.push_back(copyDesc(p.outs[0], p.outs[o], p.cnt * c.ts));
    }
    flagcxResult_t rc = R(fx_reduce_slices(plain.data(), plain.size(), 2, g->dtype, g->op, c.s));
    if (rc != flagcxSuccess) return rc;
  }
  if (!bcast.empty()) return R(fx_reduce_bcast_slices(bcast.data(), bcast.size(), 2, nout, g->dtype, g->op, c.s));
  return R(fx_copy_slices(copies.data(), copies.size(), c.s));
}

inline bool isFloating(int dtype) {
  return dtype == flagcxFloat16 || dtype == flagcxBfloat16 || dtype == flagcxFloat32 || dtype == flagcxFloat64;
}

flagcxResult_t reduceHostPieces(const Ctx &c, const std::vector<HostPiece> &pieces) {
  if ((c.g->op == flagcxMax || c.g->op == flagcxMin) && isFloating(c.g->dtype)) return chainHostPieces(c, pieces);
  std::vector<int> order;
  BcastList bcast;
  SliceList plain;
  int nout = 0;
  for (const HostPiece &p : pieces) {
    if (p.cnt == 0) continue;
    hostOrder(p.chunk, c.n, c.g->op, order);
    nout = (int)p.outs.size();
    if (c.n <= FX_MAX_SLICE_INPUTS && nout <= FX_MAX_SLICE_INPUTS) {
      if (nout == 1) {
        fxSliceDesc d;
        memset(&d, 0, sizeof(d));
        for (int j = 0; j < c.n; j++) d.in[j] = cadd(c.send(order[j]), p.off * c.ts);
        d.out = p.outs[0];
        d.count = p.cnt;
        plain.push_back(d);
      } else {
        fxBcastDesc d;
        memset(&d, 0, sizeof(d));
        for (int j = 0; j < c.n; j++) d.in[j] = cadd(c.send(order[j]), p.off * c.ts);
        for (int o = 0; o < nout; o++) d.out[o] = p.outs[o];
        d.count = p.cnt;
        bcast.push_back(d);
      }
      continue;
    }
    // more than eight ranks: one runtime-k launch per piece, then copies
    PtrList in;
    in.resize((size_t)c.n);
    for (int j = 0; j < c.n; j++) in[j] = cadd(c.send(order[j]), p.off * c.ts);
    flagcxResult_t rc = R(fx_reduce_copy(p.outs[0], in.data(), c.n, p.cnt, c.g->dtype, c.g->op, 0, c.s));
    if (rc != flagcxSuccess) return rc;
    SliceList copies;
    for (int o = 1; o < nout; o++) copies.push_back(copyDesc(p.outs[0], p.outs[o], p.cnt * c.ts));
    rc = R(fx_copy_slices(copies.data(), copies.size(), c.s));
    if (rc != flagcxSuccess) return rc;
  }
  if (!plain.empty()) {
    flagcxResult_t rc = R(fx_reduce_slices(plain.data(), plain.size(), c.n, c.g->dtype, c.g->op, c.s));
    if (rc != flagcxSuccess) return rc;
  }
  if (!bcast.empty()) return R(fx_reduce_bcast_slices(bcast.data(), bcast.size(), c.n, nout, c.g->dtype, c.g->op, c.s));
  return flagcxSuccess;
}

flagcxResult_t runAllReduce(const Ctx &c) {
  Group *g = c.g;
  const int n = c.n;
  const size_t count = g->count, ts = c.ts;
  if (n == 1) {
    if (count && c.send(0) != c.recv(0)) {
      fxSliceDesc d = copyDesc(c.send(0), c.recv(0), count * ts);
      return R(fx_copy_slices(&d, 1, c.s));
    }
    return flagcxSuccess;
  }
  if (g->order == FX_ORDER_HOST) {  // the host path's chunks and fold order; every rank receives every chunk
    std::vector<HostPiece> pieces(n);
    for (int ch = 0; ch < n; ch++) {
      pieces[ch].chunk = ch;
      hostChunk(count, n, ch, &pieces[ch].cnt, &pieces[ch].off);
      for (int r = 0; r < n; r++) pieces[ch].outs.push_back(madd(c.recv(r), pieces[ch].off * ts));
    }
    return reduceHostPieces(c, pieces);
  }
  const size_t nred = fx_nredslices(count, n, (size_t)g->nslices, (size_t)g->nredslices, (size_t)g->redslicesize);
  SliceList descs;
  if (g->algo == FX_ALGO_RING && g->op != flagcxAvg) {  // a mean is not a chain of two-input means
    // reduce-scatter: step i, rank r reduces chunk (r-i-1)%n: partial from the
    // previous rank (its sendbuff at step 0, its recvbuff afterwards) + own data.
    for (int i = 0; i < n - 1; i++) {
      for (int r = 0; r < n; r++) {
        const int prev = mod(r - 1, n), rx = mod(r - i - 1, n);
        size_t ccnt, coff;
        fx_split(count, n, rx, &ccnt, &coff);
        const void *partial = (i == 0) ? c.send(prev) : (const void *)c.recv(prev);
        flagcxResult_t rc = forPieces(g, ccnt, coff, nred, [&](size_t off, size_t, size_t cnt) {
          if (cnt == 0) return flagcxSuccess;
          fxSliceDesc d;
          memset(&d, 0, sizeof(d));
          d.in[0] = cadd(partial, off * ts);
          d.in[1] = cadd(c.send(r), off * ts);
          d.out = madd(c.recv(r), off * ts);
          d.count = cnt;
          descs.push_back(d);
          return flagcxSuccess;
        });
        if (rc != flagcxSuccess) return rc;
      }
      flagcxResult_t rc = R(fx_reduce_slices(descs.data(), descs.size(), 2, g->dtype, g->op, c.s));
      descs.clear();
      if (rc != flagcxSuccess) return rc;
    }
    // all-gather: step i, rank r receives chunk (r-i)%n from the previous rank.
    for (int i = 0; i < n - 1; i++) {
      for (int r = 0; r < n; r++) {
        const int prev = mod(r - 1, n), rx = mod(r - i, n);
        size_t ccnt, coff;
        fx_split(count, n, rx, &ccnt, &coff);
        if (ccnt) descs.push_back(copyDesc(cadd(c.recv(prev), coff * ts), madd(c.recv(r), coff * ts), ccnt * ts));
      }
      flagcxResult_t rc = R(fx_copy_slices(descs.data(), descs.size(), c.s));
      descs.clear();
      if (rc != flagcxSuccess) return rc;
    }
    return flagcxSuccess;
  }
  // direct, up to eight ranks: every piece is reduced k-way once and stored to
  // all n receive buffers by the same workgroup -- (k + n) * size bytes of
  // traffic instead of the (k + 1 + 2 (n - 1)) * size of reduce-then-copy.
  if (canBroadcast(c)) {
    BcastList bd;
    for (int ch = 0; ch < n; ch++) {
      size_t ccnt, coff;
      fx_split(count, n, ch, &ccnt, &coff);
      const int first = (g->order == FX_ORDER_RING) ? ch : 0;
      flagcxResult_t rc = forPieces(g, ccnt, coff, nred, [&](size_t off, size_t, size_t cnt) {
        if (cnt == 0) return flagcxSuccess;
        fxBcastDesc d;
        memset(&d, 0, sizeof(d));
        for (int j = 0; j < n; j++) d.in[j] = cadd(c.send(mod(first + j, n)), off * ts);
        for (int r = 0; r < n; r++) d.out[r] = madd(c.recv(r), off * ts);
        d.count = cnt;
        bd.push_back(d);
        return flagcxSuccess;
      });
      if (rc != flagcxSuccess) return rc;
    }
    return R(fx_reduce_bcast_slices(bd.data(), bd.size(), n, n, g->dtype, g->op, c.s));
  }
  // more ranks than a descriptor has slots: the runtime-k, runtime-n form of the
  // same one-read-n-stores launch.  Rank order is one launch over the whole
  // buffer; ring order starts chunk ch's fold at rank ch, one launch per chunk.
  PtrList ins;
  fx::SmallVec<void *, 16> outs;
  ins.resize((size_t)n);
  outs.resize((size_t)n);
  auto bcast = [&](size_t off, size_t cnt, int first) {
    for (int j = 0; j < n; j++) ins[j] = cadd(c.send(j), off * ts);
    for (int r = 0; r < n; r++) outs[r] = madd(c.recv(r), off * ts);
    return R(fx_reduce_bcast(outs.data(), n, ins.data(), n, cnt, g->dtype, g->op, first, c.s));
  };
  if (g->order != FX_ORDER_RING) return bcast(0, count, 0);
  if (n <= FX_MAX_INPUTS && recvsAlignedAlike(c)) {   // every chunk in one launch
    fx::SmallVec<fxChunk, 16> chunks;
    for (int ch = 0; ch < n; ch++) {
      size_t ccnt, coff;
      fx_split(count, n, ch, &ccnt, &coff);
      chunks.push_back(fxChunk{coff, coff, ccnt, ch, -1, -1});
    }
    for (int j = 0; j < n; j++) ins[j] = c.send(j);
    for (int r = 0; r < n; r++) outs[r] = c.recv(r);
    return R(fx_reduce_chunks(outs.data(), n, ins.data(), n, chunks.data(), n, g->dtype, g->op, c.s));
  }
  for (int ch = 0; ch < n; ch++) {
    size_t ccnt, coff;
    fx_split(count, n, ch, &ccnt, &coff);
    if (ccnt == 0) continue;
    const flagcxResult_t rc = bcast(coff, ccnt, ch);
    if (rc != flagcxSuccess) return rc;
  }
  return flagcxSuccess;
}

// Receive steps of tree rank a (uni_runner_impl.cc:1314-1326): the root takes
// ceil(log2 n); others ctz(a), clipped so that a + 2^i stays below n.
int treeSteps(int a, int n) {
  int total = 0;
  while ((1 << total) < n) total++;
  if (a == 0) return total;
  int st = __builtin_ctz((unsigned)a);
  if (st && n - a <= (1 << (st - 1))) {
    int rest = n - a - 1;
    for (st = 0; rest; rest >>= 1) st++;
  }
  return st;
}

flagcxResult_t runReduce(const Ctx &c) {
  Group *g = c.g;
  const int n = c.n, root = g->root;
  const size_t count = g->count, ts = c.ts;
  if (count == 0) return flagcxSuccess;
  if (g->order == FX_ORDER_HOST && n > 1) {  // the host path reduce-scatters, then gathers the chunks on the root
    std::vector<HostPiece> pieces(n);
    for (int ch = 0; ch < n; ch++) {
      pieces[ch].chunk = ch;
      hostChunk(count, n, ch, &pieces[ch].cnt, &pieces[ch].off);
      pieces[ch].outs.push_back(madd(c.recv(root), pieces[ch].off * ts));
    }
    return reduceHostPieces(c, pieces);
  }
  if (g->order != FX_ORDER_TREE || n == 1 || g->op == flagcxAvg) {
    PtrList in;
    in.resize((size_t)n);
    for (int j = 0; j < n; j++) in[j] = c.send(j);
    return R(fx_reduce_copy(c.recv(root), in.data(), n, count, g->dtype, g->op, 0, c.s));
  }
  // Tree order: round i, every tree rank a with more than i receive steps
  // computes partial(a) = partial(a + 2^i) (op) partial(a).  Up to eight ranks
  // that is one launch that keeps the partials in registers (in[a] = tree rank
  // a's data); beyond, partials live in a per-rank scratch row, one launch per
  // round, and the root's last round writes recvbuff.
  if (n <= FX_MAX_SLICE_INPUTS) {
    fxBcastDesc d;
    memset(&d, 0, sizeof(d));
    for (int a = 0; a < n; a++) d.in[a] = c.send(mod(a + root, n));
    d.out[0] = c.recv(root);
    d.count = count;
    return R(fx_reduce_ordered(&d, 1, n, 1, g->dtype, g->op, FX_FOLD_TREE, c.s));
  }
  flagcxResult_t rc = ensureScratch(g, (size_t)n * count * ts, c.s);
  if (rc != flagcxSuccess) return rc;
  const int total = treeSteps(0, n);
  auto rankOf = [&](int a) { return mod(a + root, n); };
  auto partial = [&](int a, int round) -> const void * {   // where tree rank a's partial is before `round`
    return (round == 0 || treeSteps(a, n) == 0) ? c.send(rankOf(a)) : madd(g->scratch, (size_t)a * count * ts);
  };
  SliceList descs;
  for (int i = 0; i < total; i++) {
    for (int a = 0; a < n; a++) {
      if (treeSteps(a, n) <= i) continue;
      fxSliceDesc d;
      memset(&d, 0, sizeof(d));
      d.in[0] = partial(a + (1 << i), i);   // received
      d.in[1] = partial(a, i);              // own
      d.out = (a == 0 && i == total - 1) ? c.recv(root) : madd(g->scratch, (size_t)a * count * ts);
      d.count = count;
      descs.push_back(d);
    }
    rc = R(fx_reduce_slices(descs.data(), descs.size(), 2, g->dtype, g->op, c.s));
    descs.clear();
    if (rc != flagcxSuccess) return rc;
  }
  return flagcxSuccess;
}

flagcxResult_t runReduceScatter(const Ctx &c) {
  Group *g = c.g;
  const int n = c.n;
  const size_t rcount = g->count, ts = c.ts;
  if (n == 1) {
    if (rcount && c.send(0) != c.recv(0)) {
      fxSliceDesc d = copyDesc(c.send(0), c.recv(0), rcount * ts);
      return R(fx_copy_slices(&d, 1, c.s));
    }
    return flagcxSuccess;
  }
  if (g->order == FX_ORDER_HOST) {  // chunk r = [r * recvcount, (r+1) * recvcount) ends on rank r
    std::vector<HostPiece> pieces(n);
    for (int r = 0; r < n; r++) {
      pieces[r].chunk = r;
      pieces[r].off = (size_t)r * rcount;
      pieces[r].cnt = rcount;
      pieces[r].outs.push_back(c.recv(r));
    }
    return reduceHostPieces(c, pieces);
  }
  const size_t nred = fx_nredslices(rcount, n, (size_t)g->nslices, (size_t)g->nredslices, (size_t)g->redslicesize);
  SliceList descs;
  KwayRun run;
  if (g->algo == FX_ALGO_RING && g->op != flagcxAvg) {  // a mean is not a chain of two-input means
    // Per-rank scratch of n*recvcount elements holds the travelling partials.
    flagcxResult_t rc = ensureScratch(g, (size_t)n * n * rcount * ts, c.s);
    if (rc != flagcxSuccess) return rc;
    auto scratch = [&](int r) { return madd(g->scratch, (size_t)r * n * rcount * ts); };
    for (int i = 0; i < n - 1; i++) {
      for (int r = 0; r < n; r++) {
        const int prev = mod(r - 1, n), rx = mod(r - i - 2, n);
        const void *partial = (i == 0) ? c.send(prev) : (const void *)scratch(prev);
        rc = forPieces(g, rcount, (size_t)rx * rcount, nred, [&](size_t off, size_t inSlice, size_t cnt) {
          if (cnt == 0) return flagcxSuccess;
          fxSliceDesc d;
          memset(&d, 0, sizeof(d));
          d.in[0] = cadd(partial, off * ts);
          d.in[1] = cadd(c.send(r), off * ts);
          d.out = (i == n - 2) ? madd(c.recv(r), inSlice * ts) : madd(scratch(r), off * ts);
          d.count = cnt;
          descs.push_back(d);
          return flagcxSuccess;
        });
        if (rc != flagcxSuccess) return rc;
      }
      rc = R(fx_reduce_slices(descs.data(), descs.size(), 2, g->dtype, g->op, c.s));
      descs.clear();
      if (rc != flagcxSuccess) return rc;
    }
    return flagcxSuccess;
  }
  if (n > FX_MAX_SLICE_INPUTS && n <= FX_MAX_INPUTS) {   // chunk r of every send buffer onto rank r, all in one launch
    fx::SmallVec<fxChunk, 16> chunks;
    PtrList ins;
    fx::SmallVec<void *, 16> outs;
    for (int r = 0; r < n; r++) {
      chunks.push_back(fxChunk{(size_t)r * rcount, 0, rcount, (g->order == FX_ORDER_RING) ? mod(r + 1, n) : 0, -1, r});
      ins.push_back(c.send(r));
      outs.push_back(c.recv(r));
    }
    return R(fx_reduce_chunks(outs.data(), n, ins.data(), n, chunks.data(), n, g->dtype, g->op, c.s));
  }
  for (int r = 0; r < n; r++) {
    const int first = (g->order == FX_ORDER_RING) ? mod(r + 1, n) : 0;
    flagcxResult_t rc = forPieces(g, rcount, (size_t)r * rcount, nred, [&](size_t off, size_t inSlice, size_t cnt) {
      return kway(c, descs, run, off, cnt, madd(c.recv(r), inSlice * ts), first);
    });
    if (rc != flagcxSuccess) return rc;
  }
  return flushKway(c, descs, run);
}

flagcxResult_t runAllGather(const Ctx &c) {
  const size_t bytes = c.g->count * c.ts;
  if (bytes == 0) return flagcxSuccess;
  if (canBroadcast(c)) {  // each rank's block is read once and stored to every receive buffer
    BcastList bd;
    bd.resize((size_t)c.n);
    for (int r = 0; r < c.n; r++) {
      memset(&bd[r], 0, sizeof(fxBcastDesc));
      bd[r].in[0] = c.send(r);
      for (int j = 0; j < c.n; j++) bd[r].out[j] = madd(c.recv(j), (size_t)r * bytes);
      bd[r].count = bytes;
    }
    return R(fx_reduce_bcast_slices(bd.data(), bd.size(), 1, c.n, 0, -1, c.s));
  }
  if (c.n <= FX_MAX_INPUTS && recvsAlignedAlike(c)) {   // rank q's block into slot q of every rank, all in one launch
    fx::SmallVec<fxChunk, 16> chunks;
    PtrList ins;
    fx::SmallVec<void *, 16> outs;
    for (int q = 0; q < c.n; q++) {
      chunks.push_back(fxChunk{0, (size_t)q * bytes, bytes, 0, q, -1});
      ins.push_back(c.send(q));
      outs.push_back(c.recv(q));
    }
    return R(fx_reduce_chunks(outs.data(), c.n, ins.data(), c.n, chunks.data(), c.n, 0, -1, c.s));
  }
  SliceList descs;
  for (int r = 0; r < c.n; r++)
    for (int j = 0; j < c.n; j++) {
      void *dst = madd(c.recv(j), (size_t)r * bytes);
      if (dst != c.send(r)) descs.push_back(copyDesc(c.send(r), dst, bytes));
    }
  return R(fx_copy_slices(descs.data(), descs.size(), c.s));
}

// When no receive segment overlaps any send segment, every segment goes
// straight from the sender's buffer to the receiver's: one batched launch.
// Otherwise (in-place use) every rank's segments are packed into contiguous
// staging slots and unpacked from the peers' slots: two launches.
flagcxResult_t runAlltoAllv(const Ctx &c) {
  Group *g = c.g;
  const int n = c.n;
  const size_t ts = c.ts;
  std::vector<size_t> base(n + 1, 0);
  struct Range {
    uintptr_t lo, hi;
  };
  std::vector<Range> sendR, recvR;
  for (int r = 0; r < n; r++) {
    size_t tot = 0;
    for (int i = 0; i < n; i++) {
      const size_t cnt = g->posts[r].sendcounts[i];
      if (cnt != g->posts[i].recvcounts[r]) return flagcxInvalidArgument;
      tot += cnt;
      if (cnt && (!c.send(r) || !c.recv(i))) return flagcxInvalidArgument;
      if (cnt) {
        const uintptr_t s = (uintptr_t)c.send(r) + g->posts[r].sdispls[i] * ts;
        const uintptr_t d = (uintptr_t)c.recv(i) + g->posts[i].rdispls[r] * ts;
        sendR.push_back({s, s + cnt * ts});
        recvR.push_back({d, d + cnt * ts});
      }
    }
    base[r + 1] = base[r] + ((tot * ts + 255) & ~(size_t)255);
  }
  if (base[n] == 0) return flagcxSuccess;
  // Does any receive segment overlap any send segment?  First by rank: the span of all a rank sends against the
  // span of all a rank receives (n * n pairs instead of one per pair of segments); only where two spans meet, by
  // segment, in address order.
  bool overlap = false;
  {
    std::vector<Range> sendSpan(n, Range{UINTPTR_MAX, 0}), recvSpan(n, Range{UINTPTR_MAX, 0});
    size_t at = 0;
    for (int r = 0; r < n; r++)
      for (int i = 0; i < n; i++) {
        if (!g->posts[r].sendcounts[i]) continue;
        const Range &sr = sendR[at], &rr = recvR[at];   // pushed pairwise above: rank r's segment for rank i, and where it lands
        at++;
        sendSpan[r].lo = std::min(sendSpan[r].lo, sr.lo);
        sendSpan[r].hi = std::max(sendSpan[r].hi, sr.hi);
        recvSpan[i].lo = std::min(recvSpan[i].lo, rr.lo);
        recvSpan[i].hi = std::max(recvSpan[i].hi, rr.hi);
      }
    bool spansMeet = false;
    for (int r = 0; r < n && !spansMeet; r++)
      for (int i = 0; i < n && !spansMeet; i++)
        spansMeet = recvSpan[i].lo < sendSpan[r].hi && sendSpan[r].lo < recvSpan[i].hi;
    if (spansMeet) {
      struct Tagged {
        uintptr_t lo, hi;
        int recv;
      };
      std::vector<Tagged> all;
      all.reserve(sendR.size() + recvR.size());
      for (const Range &x : sendR) all.push_back(Tagged{x.lo, x.hi, 0});
      for (const Range &x : recvR) all.push_back(Tagged{x.lo, x.hi, 1});
      std::sort(all.begin(), all.end(), [](const Tagged &a, const Tagged &b) { return a.lo < b.lo; });
      uintptr_t reach[2] = {0, 0};   // how far the segments of either kind seen so far extend
      for (const Tagged &x : all) {
        if (reach[1 - x.recv] > x.lo) {
          overlap = true;
          break;
        }
        reach[x.recv] = std::max(reach[x.recv], x.hi);
      }
    }
  }
  if (!overlap) {
    SliceList direct;
    for (size_t a = 0; a < recvR.size(); a++)
      direct.push_back(copyDesc((const void *)sendR[a].lo, (void *)recvR[a].lo, recvR[a].hi - recvR[a].lo));
    return R(fx_copy_slices(direct.data(), direct.size(), c.s));
  }
  flagcxResult_t rc = ensureScratch(g, base[n], c.s);
  if (rc != flagcxSuccess) return rc;
  SliceList pack, unpack;
  for (int r = 0; r < n; r++) {
    size_t slot = 0;
    for (int i = 0; i < n; i++) {
      const size_t cnt = g->posts[r].sendcounts[i];
      if (cnt) {
        void *stage = madd(g->scratch, base[r] + slot * ts);
        pack.push_back(copyDesc(cadd(c.send(r), g->posts[r].sdispls[i] * ts), stage, cnt * ts));
        unpack.push_back(copyDesc(stage, madd(c.recv(i), g->posts[i].rdispls[r] * ts), cnt * ts));
      }
      slot += cnt;
    }
  }
  rc = R(fx_copy_slices(pack.data(), pack.size(), c.s));
  if (rc != flagcxSuccess) return rc;
  return R(fx_copy_slices(unpack.data(), unpack.size(), c.s));
}

// gather / scatter / broadcast / alltoall move bytes only: one batched copy
// launch each (the reference builds them from grouped send/recv pairs,
// flagcx/adaptor/ccl/rccl_adaptor.cc:126-184,222-246).
flagcxResult_t runGather(const Ctx &c) {
  const size_t bytes = c.g->count * c.ts;
  SliceList d;
  for (int r = 0; r < c.n && bytes; r++) {
    void *dst = madd(c.recv(c.g->root), (size_t)r * bytes);
    if (dst != c.send(r)) d.push_back(copyDesc(c.send(r), dst, bytes));
  }
  return R(fx_copy_slices(d.data(), d.size(), c.s));
}

flagcxResult_t runScatter(const Ctx &c) {
  const size_t bytes = c.g->count * c.ts;
  SliceList d;
  for (int r = 0; r < c.n && bytes; r++) {
    const void *src = cadd(c.send(c.g->root), (size_t)r * bytes);
    if (src != c.recv(r)) d.push_back(copyDesc(src, c.recv(r), bytes));
  }
  return R(fx_copy_slices(d.data(), d.size(), c.s));
}

flagcxResult_t runBroadcast(const Ctx &c) {
  const size_t bytes = c.g->count * c.ts;
  if (bytes && canBroadcast(c)) {
    fxBcastDesc b;
    memset(&b, 0, sizeof(b));
    b.in[0] = c.send(c.g->root);
    for (int r = 0; r < c.n; r++) b.out[r] = c.recv(r);
    b.count = bytes;
    return R(fx_reduce_bcast_slices(&b, 1, 1, c.n, 0, -1, c.s));
  }
  if (bytes && c.n <= FX_MAX_INPUTS) {   // more ranks: the run-time form of the same one-read-n-stores copy
    fx::SmallVec<void *, 16> outs;
    for (int r = 0; r < c.n; r++) outs.push_back(c.recv(r));
    const void *src = c.send(c.g->root);
    return R(fx_reduce_bcast(outs.data(), c.n, &src, 1, bytes, 0, -1, 0, c.s));
  }
  SliceList d;
  for (int r = 0; r < c.n && bytes; r++)
    if (c.recv(r) != c.send(c.g->root)) d.push_back(copyDesc(c.send(c.g->root), c.recv(r), bytes));
  return R(fx_copy_slices(d.data(), d.size(), c.s));
}

// Block i of rank r's sendbuff becomes block r of rank i's recvbuff.  The
// one-launch kernel reads and writes concurrently, so if ANY rank's send buffer
// meets ANY rank's receive buffer (a rank in place, rank a receiving into what
// rank b sends, a partial overlap) the blocks go through staging first.
flagcxResult_t runAlltoAll(const Ctx &c) {
  Group *g = c.g;
  const int n = c.n;
  const size_t bytes = g->count * c.ts;
  if (bytes == 0) return flagcxSuccess;
  bool inplace = false;
  const size_t span = (size_t)n * bytes;
  for (int r = 0; r < n && !inplace; r++)
    for (int i = 0; i < n && !inplace; i++) {
      const uintptr_t s = (uintptr_t)c.send(r), d = (uintptr_t)c.recv(i);
      inplace = s < d + span && d < s + span;
    }
  SliceList d;
  if (!inplace) {   // every block straight from its sender to its receiver, one launch
    PtrList sends;
    fx::SmallVec<void *, 16> recvs;
    for (int r = 0; r < n; r++) {
      sends.push_back(c.send(r));
      recvs.push_back(c.recv(r));
    }
    return R(fx_alltoall(recvs.data(), sends.data(), n, bytes, c.s));
  }
  flagcxResult_t rc = ensureScratch(g, (size_t)n * n * bytes, c.s);
  if (rc != flagcxSuccess) return rc;
  for (int r = 0; r < n; r++)
    d.push_back(copyDesc(c.send(r), madd(g->scratch, (size_t)r * n * bytes), (size_t)n * bytes));
  rc = R(fx_copy_slices(d.data(), d.size(), c.s));
  if (rc != flagcxSuccess) return rc;
  PtrList staged;
  fx::SmallVec<void *, 16> recvs;
  for (int r = 0; r < n; r++) {
    staged.push_back(cadd(g->scratch, (size_t)r * n * bytes));
    recvs.push_back(c.recv(r));
  }
  return R(fx_alltoall(recvs.data(), staged.data(), n, bytes, c.s));
}

flagcxResult_t runCustomAllReduce(const Ctx &c) {
  Group *g = c.g;
  if (g->count == 0) return flagcxSuccess;
  {  // stage every rank's sendbuff into its window unless it already is the window
    SliceList stage;
    for (int r = 0; r < c.n; r++)
      if (c.send(r) != g->windows[r]) stage.push_back(copyDesc(c.send(r), g->windows[r], g->count * c.ts));
    if (!stage.empty()) {
      const flagcxResult_t rc = R(fx_copy_slices(stage.data(), stage.size(), c.s));
      if (rc != flagcxSuccess) return rc;
    }
  }
  if (canBroadcast(c)) {  // every rank's result is the same fold of the windows: compute it once
    fxBcastDesc b;
    memset(&b, 0, sizeof(b));
    for (int j = 0; j < c.n; j++) b.in[j] = g->windows[j];
    for (int r = 0; r < c.n; r++) b.out[r] = c.recv(r);
    b.count = g->count;
    return R(fx_reduce_bcast_slices(&b, 1, c.n, c.n, g->dtype, g->op, c.s));
  }
  fx::SmallVec<void *, 16> outs;
  outs.resize((size_t)c.n);
  for (int r = 0; r < c.n; r++) outs[r] = c.recv(r);
  return R(fx_reduce_bcast(outs.data(), c.n, (const void *const *)g->windows.data(), c.n, g->count, g->dtype, g->op, 0,
                           c.s));
}

}  // namespace fxsim
