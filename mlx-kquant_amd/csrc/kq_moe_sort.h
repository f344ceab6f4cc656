// Pair sort of the batched MoE ops, shared by the launchers that fold it into their own prologue kernel.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace kqsort {

constexpr int SEG_M = 32;  // pairs per segment at most
constexpr int SORT_MAX_E = 4096;

struct Segment {
  int expert, start, count, pad;
};

// ------------------------------------------------------------------ pair sort (one workgroup)
// order[] = pair ids grouped by expert; segs[] = (expert, first position in order, pairs <= 32).
// Pairs whose expert id is out of range are left out (their output rows are not written).
// One pass over the indices: a pair's rank inside its expert is what the histogram's atomic add returns, so the
// scatter needs no second count (the order inside an expert is then arbitrary, which no consumer depends on: every
// pair's output row is its own).  The scans over the experts run as wave scans with one barrier.  Up to 8 pairs per
// thread stay in registers; larger inputs take a second pass over the indices.
template <int THREADS>
__device__ __forceinline__ void moe_sort_body(const uint32_t* __restrict__ idx, int P, int E, int* __restrict__ order,
                                              Segment* __restrict__ segs, int* __restrict__ nseg_out, int* cnt,
                                              int* scan_p, int* scan_s) {
  constexpr int PPT = 8, NW = THREADS / 64;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const bool small = P <= THREADS * PPT;
  for (int e = tid; e < E; e += THREADS) cnt[e] = 0;
  __syncthreads();
  uint32_t ev[PPT];
  int rk[PPT];
  if (small) {
#pragma unroll
    for (int i = 0; i < PPT; i++) {
      const int p = tid + THREADS * i;
      ev[i] = p < P ? idx[p] : 0xffffffffu;
    }
#pragma unroll
    for (int i = 0; i < PPT; i++) rk[i] = ev[i] < (uint32_t)E ? atomicAdd(&cnt[ev[i]], 1) : -1;
  } else {
    for (int p = tid; p < P; p += THREADS) {
      const uint32_t e = idx[p];
      if (e < (uint32_t)E) atomicAdd(&cnt[e], 1);
    }
  }
  __syncthreads();
  // exclusive scans of pair counts and segment counts: thread t owns experts [t*ch, t*ch + ch)
  const int ch = (E + THREADS - 1) / THREADS;
  int lp = 0, ls = 0;
  for (int i = 0; i < ch; i++) {
    const int e = tid * ch + i;
    if (e < E) {
      lp += cnt[e];
      ls += (cnt[e] + SEG_M - 1) / SEG_M;
    }
  }
  int ip = lp, is = ls;  // inclusive scan inside the wave
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int vp = __shfl_up(ip, off), vs = __shfl_up(is, off);
    if (lane >= off) {
      ip += vp;
      is += vs;
    }
  }
  if (lane == 63) {
    scan_p[wave] = ip;
    scan_s[wave] = is;
  }
  __syncthreads();
  int wp = 0, ws = 0, tp = 0, ts = 0;
#pragma unroll
  for (int wv = 0; wv < NW; wv++) {
    const int vp = scan_p[wv], vs = scan_s[wv];
    if (wv < wave) {
      wp += vp;
      ws += vs;
    }
    tp += vp;
    ts += vs;
  }
  (void)tp;
  int bp = wp + ip - lp, bs = ws + is - ls;  // exclusive prefix of this thread's experts
  if (tid == 0) *nseg_out = ts;
  for (int i = 0; i < ch; i++) {
    const int e = tid * ch + i;
    if (e < E) {
      const int c = cnt[e];
      for (int k = 0, sg = bs; k < c; k += SEG_M, sg++) segs[sg] = Segment{e, bp + k, c - k < SEG_M ? c - k : SEG_M, 0};
      bs += (c + SEG_M - 1) / SEG_M;
      cnt[e] = bp;  // first position of the expert's pairs (small) / running cursor
      bp += c;
    }
  }
  __syncthreads();
  if (small) {
#pragma unroll
    for (int i = 0; i < PPT; i++)
      if (rk[i] >= 0) order[cnt[ev[i]] + rk[i]] = tid + THREADS * i;
  } else {
    for (int p = tid; p < P; p += THREADS) {
      const uint32_t e = idx[p];
      if (e < (uint32_t)E) order[atomicAdd(&cnt[e], 1)] = p;
    }
  }
}

}  // namespace kqsort
