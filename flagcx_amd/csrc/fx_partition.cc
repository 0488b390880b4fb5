// The reference's chunk / slice / red-slice partition as node lists: what its
// uniRunner builds as reduce nodes for one rank
// (flagcx/runner/uni_runner_impl.cc:82-157 LocRed, :661-1007 sliced ring
// all-reduce, :1009-1264 ring reduce-scatter).  Buffer ids: 0 = sendbuff,
// 1 = recvbuff, 2 = scratch; offsets and counts in elements.
#include "flagcx_amd/fx_kernels.h"
#include "flagcx_amd/fx_sim.h"

namespace {

inline int mod(int a, int n) { return ((a % n) + n) % n; }

void partNode(fxRedNode *n, int step, int rank, size_t slice, int in1, int in2, int out, size_t inOff, size_t outOff,
              size_t cnt) {
  n->step = step;
  n->rank = rank;
  n->slice = (int32_t)slice;
  n->in1_buf = in1;
  n->in2_buf = in2;
  n->out_buf = out;
  n->in1_off = n->in2_off = inOff;
  n->out_off = outOff;
  n->count = cnt;
}

}  // namespace

extern "C" {
#pragma GCC visibility push(default)

size_t fx_part_ring_ar(size_t count, int nranks, int rank, size_t nslices, size_t nred, fxRedNode *nodes) {
  if (nranks < 2 || nslices == 0 || nred == 0) return 0;
  size_t w = 0;
  for (size_t s = 0; s < nslices; s++)
    for (int i = 0; i < nranks - 1; i++) {
      size_t ccnt, coff, scnt, soff;
      fx_split(count, nranks, mod(rank - i - 1, nranks), &ccnt, &coff);
      fx_split(ccnt, nslices, s, &scnt, &soff);
      for (size_t q = 0; q < nred; q++, w++) {
        size_t rcnt, roff;
        fx_split(scnt, nred, q, &rcnt, &roff);
        if (nodes) partNode(&nodes[w], i, rank, s, 1, 0, 1, coff + soff + roff, coff + soff + roff, rcnt);
      }
    }
  return w;
}

size_t fx_part_ring_rs(size_t recvcount, int nranks, int rank, size_t nslices, size_t nred, fxRedNode *nodes) {
  if (nranks < 2 || nslices == 0 || nred == 0) return 0;
  size_t w = 0;
  for (size_t s = 0; s < nslices; s++)
    for (int i = 0; i < nranks - 1; i++) {
      const size_t coff = (size_t)mod(rank - i - 2, nranks) * recvcount;
      size_t scnt, soff;
      fx_split(recvcount, nslices, s, &scnt, &soff);
      for (size_t q = 0; q < nred; q++, w++) {
        size_t rcnt, roff;
        fx_split(scnt, nred, q, &rcnt, &roff);
        if (!nodes) continue;
        const bool last = (i == nranks - 2);
        partNode(&nodes[w], i, rank, s, 2, 0, last ? 1 : 2, coff + soff + roff, last ? soff + roff : coff + soff + roff,
                 rcnt);
      }
    }
  return w;
}

size_t fx_part_locred(size_t count, int nranks, int rank, size_t nslices, fxRedNode *nodes) {
  if (nranks < 2 || nslices == 0) return 0;
  size_t ccnt, coff;
  fx_split(count, nranks, rank, &ccnt, &coff);
  for (size_t s = 0; s < nslices && nodes; s++) {
    size_t scnt, soff;
    fx_split(ccnt, nslices, s, &scnt, &soff);
    partNode(&nodes[s], 0, rank, s, 1, 0, 1, coff + soff, coff + soff, scnt);
  }
  return nslices;
}

#pragma GCC visibility pop
}  // extern "C"
