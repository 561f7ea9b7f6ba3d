// Device helpers shared by the trajectory kernels: cross-lane reductions, the activation, likelihood
// and prior terms, agent-scope accesses, the per-wave step context and the bounded group barrier.
#pragma once

#include <hip/hip_runtime.h>

#include "bnn_device.h"
#include "bnn_rng.h"

namespace bnn {

typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f2 __attribute__((ext_vector_type(2)));

// ------------------------------------------------------------------------------------------------
// small device helpers
// ------------------------------------------------------------------------------------------------
// The thread index as a value the compiler cannot see through.  Indices and addresses derived from
// it are computed where they are used, every time: derived from threadIdx.x they are invariant across
// the leapfrog steps, get hoisted out of the step loop, and then sit in registers across the tile
// loop, which has none to spare.
__device__ __forceinline__ int opaque_tid() {
  int t = (int)threadIdx.x;
  asm volatile("" : "+v"(t));
  return t;
}

// A point all values of a row of `v` must have reached before anything computed from them starts (one
// assembly statement that takes them all): placed between a batch of loads and the arithmetic on them,
// it keeps the compiler from reading and adding one value at a time (a chain of load latencies).
template <int A, int B>
__device__ __forceinline__ void keep_together(float (&v)[A][B]) {
  static_assert(B == 4 || B == 8 || B == 12 || B == 16, "rows of 4, 8, 12 or 16 values");
#pragma unroll
  for (int i = 0; i < A; ++i) {
    float(&r)[B] = v[i];
    if constexpr (B == 4) {
      asm volatile("" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]));
    } else if constexpr (B == 8) {
      asm volatile("" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]));
    } else if constexpr (B == 12) {
      asm volatile("" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]),
                        "+v"(r[8]), "+v"(r[9]), "+v"(r[10]), "+v"(r[11]));
    } else {
      // an assembly statement takes at most 30 operands (a read-write one counts twice)
      asm volatile("" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]),
                        "+v"(r[8]), "+v"(r[9]), "+v"(r[10]), "+v"(r[11]), "+v"(r[12]), "+v"(r[13]), "+v"(r[14]));
      asm volatile("" : "+v"(r[15]));
    }
  }
}

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

// sum over the 16 lanes of a DPP row; every lane of the row receives the same bits (each step adds
// a value to its mirror image, and a + b == b + a)
__device__ __forceinline__ float row16_allreduce(float v) {
  v += dpp_move<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_move<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_move<0x141>(v);  // row_half_mirror
  v += dpp_move<0x140>(v);  // row_mirror
  return v;
}
// the same for a double (its two halves moved separately)
template <int CTRL>
__device__ __forceinline__ double dpp_move_d(double v) {
  const unsigned long long b = __builtin_bit_cast(unsigned long long, v);
  const unsigned lo = (unsigned)__builtin_amdgcn_update_dpp(0, (int)(unsigned)b, CTRL, 0xf, 0xf, true);
  const unsigned hi = (unsigned)__builtin_amdgcn_update_dpp(0, (int)(unsigned)(b >> 32), CTRL, 0xf, 0xf, true);
  return __builtin_bit_cast(double, ((unsigned long long)hi << 32) | lo);
}
__device__ __forceinline__ double row16_allreduce_d(double v) {
  v += dpp_move_d<0xB1>(v);
  v += dpp_move_d<0x4E>(v);
  v += dpp_move_d<0x141>(v);
  v += dpp_move_d<0x140>(v);
  return v;
}
// Four sums over the 16 lanes of a DPP row at once, in 8 instructions instead of 4 x 4: the four
// values are first folded into each other across the four banks of four lanes (writes masked by
// bank), so that bank j of the result holds the sum of v_j -- the same bits in its four lanes (the
// last two steps add a value to its mirror image).  row16_bcast<j> then hands bank j to all 16 lanes.
// Written in assembly because a bank-masked DPP add has no builtin; a DPP instruction must not read a
// register the instruction before it (or the one before that) wrote, hence the s_nops.
__device__ __forceinline__ float row16_reduce4(float v0, float v1, float v2, float v3) {
  float r01, r23, z;
  asm("s_nop 1\n\t"
      "v_add_f32_dpp %[r01], %[v0], %[v0] row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %[r23], %[v2], %[v2] row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %[r01], %[v1], %[v1] row_half_mirror row_mask:0xf bank_mask:0xa\n\t"
      "v_add_f32_dpp %[r23], %[v3], %[v3] row_half_mirror row_mask:0xf bank_mask:0xa\n\t"
      "s_nop 0\n\t"
      "v_add_f32_dpp %[z], %[r01], %[r01] row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_add_f32_dpp %[z], %[r23], %[r23] row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
      "s_nop 1\n\t"
      "v_add_f32_dpp %[z], %[z], %[z] quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 1\n\t"
      "v_add_f32_dpp %[z], %[z], %[z] quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf"
      : [r01] "=&v"(r01), [r23] "=&v"(r23), [z] "=&v"(z)
      : [v0] "v"(v0), [v1] "v"(v1), [v2] "v"(v2), [v3] "v"(v3));
  return z;
}
template <int J>
__device__ __forceinline__ float row16_bcast(float z) {
  return dpp_move<0x150 + 4 * J>(z);  // row_newbcast: lane 4 J of each row to its 16 lanes
}

// sum over the 8 lanes of a half row
__device__ __forceinline__ float row8_allreduce(float v) {
  v += dpp_move<0xB1>(v);
  v += dpp_move<0x4E>(v);
  v += dpp_move<0x141>(v);
  return v;
}

__device__ __forceinline__ double shfl_xor_d(double v, int mask) {
  const uint64_t b = double_to_bits(v);
  const uint32_t lo = (uint32_t)__shfl_xor((int)(uint32_t)b, mask);
  const uint32_t hi = (uint32_t)__shfl_xor((int)(uint32_t)(b >> 32), mask);
  return bits_to_double(((uint64_t)hi << 32) | lo);
}

__device__ __forceinline__ unsigned long long shfl_xor_u64(unsigned long long b, int mask) {
  const uint32_t lo = (uint32_t)__shfl_xor((int)(uint32_t)b, mask);
  const uint32_t hi = (uint32_t)__shfl_xor((int)(uint32_t)(b >> 32), mask);
  return ((unsigned long long)hi << 32) | lo;
}

// State hash of a workgroup.  Every workgroup of a chain group integrates the same parameters from
// the same exchanged gradients and must hold the same bits; each folds what it holds into a 64-bit
// value per thread (fold_hash), the values of a workgroup are added up when the kernel ends
// (publish_hash) and the host compares the workgroups of a group.  A workgroup that ever read a
// stale partial record ends with a different hash.
__device__ __forceinline__ unsigned long long fold_hash(unsigned long long h, float a, float b) {
  return mix64(h ^ (((unsigned long long)__builtin_bit_cast(uint32_t, a) << 32) |
                    __builtin_bit_cast(uint32_t, b)));
}
// s_tmp: one slot per wave.  Contains two workgroup barriers: call from uniform control flow.
__device__ __forceinline__ void publish_hash(unsigned long long h, unsigned long long* s_tmp, int n_waves,
                                             unsigned long long* dst, bool perturb) {
#pragma unroll
  for (int msk = 1; msk < 64; msk <<= 1) h += shfl_xor_u64(h, msk);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) s_tmp[threadIdx.x >> 6] = h;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned long long tot = 0;
    for (int wv = 0; wv < n_waves; ++wv) tot += s_tmp[wv];
    *dst = perturb ? tot ^ 1ull : tot;
  }
}

// activation of the hidden layer, include/mcmc/kernel_helpers.h:34-42:
// tanh(x) = 2 sigmoid(2x) - 1 with e^(-2x) = 2^(x * -2/ln 2); identity below the cutoff
__device__ __forceinline__ float tanh_fwd(float x) {
  const float e = __builtin_amdgcn_exp2f(x * -2.88539008177792681472f);
  const float sigm = __builtin_amdgcn_rcpf(1.0f + e);
  const float r = __builtin_fmaf(sigm, 2.0f, -1.0f);
  return __builtin_fabsf(x) < 0.0048176045529544353485f ? x : r;
}

// per-row log-likelihood gradient (and value) given the residual, mcmc_step_ffma.h:293-301
template <int LIK>
__device__ __forceinline__ float lik_grad(const ModelConsts& mc, float resid, float& diff_out) {
  const float diff = resid * mc.scale_recp;
  diff_out = diff;
  if (LIK == 0) {
    return diff * mc.g_scale * __builtin_amdgcn_rcpf(__builtin_fmaf(diff, diff, mc.df));
  } else {
    return diff * mc.scale_recp;
  }
}
template <int LIK>
__device__ __forceinline__ float lik_value(const ModelConsts& mc, float diff) {
  if (LIK == 0) {
    return mc.l_scale * log1pf(diff * diff * mc.df_recp) - mc.lik_norm;
  } else {
    return -0.5f * (diff * diff) - mc.lik_norm;
  }
}

// prior terms, mcmc_step_ffma.h:113-118
__device__ __forceinline__ float prior_logp(const ModelConsts& mc, float w) {
  const float lp = w * mc.prior_recp;
  return -(lp * lp) * 0.5f - mc.prior_norm;
}
__device__ __forceinline__ float prior_grad(const ModelConsts& mc, float w) {
  return w * mc.prior_neg_recp2;
}

__device__ __forceinline__ float ld_agent(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_agent(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Eight 16-byte agent-scope loads in flight at once, collected before the statement ends: the loads
// and the wait form ONE assembly statement, so the compiler sees the eight results as defined only
// once they have landed (it may spill or copy them afterwards like any other value).  The results are
// early-clobber: a returning load must not land in a register that still holds the address of a load
// not yet issued.  Every address must be valid; callers clamp out-of-range records to a valid one and
// discard the value.
__device__ __forceinline__ void ld_agent4x8(f4 (&t)[8], const float* const (&p)[8]) {
  asm volatile(
      "global_load_dwordx4 %0, %8, off sc1\n\t"
      "global_load_dwordx4 %1, %9, off sc1\n\t"
      "global_load_dwordx4 %2, %10, off sc1\n\t"
      "global_load_dwordx4 %3, %11, off sc1\n\t"
      "global_load_dwordx4 %4, %12, off sc1\n\t"
      "global_load_dwordx4 %5, %13, off sc1\n\t"
      "global_load_dwordx4 %6, %14, off sc1\n\t"
      "global_load_dwordx4 %7, %15, off sc1\n\t"
      "s_waitcnt vmcnt(0)"
      : "=&v"(t[0]), "=&v"(t[1]), "=&v"(t[2]), "=&v"(t[3]), "=&v"(t[4]), "=&v"(t[5]), "=&v"(t[6]),
        "=&v"(t[7])
      : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]), "v"(p[7])
      : "memory");
}

// the same with N = 1, 2 or 4 loads (the addresses p[N ..] are not touched)
template <int N>
__device__ __forceinline__ void ld_agent4xN(f4 (&t)[8], const float* const (&p)[8]) {
  static_assert(N == 1 || N == 2 || N == 4 || N == 8, "1, 2, 4 or 8 loads");
  if constexpr (N == 8) {
    ld_agent4x8(t, p);
  } else if constexpr (N == 4) {
    asm volatile(
        "global_load_dwordx4 %0, %4, off sc1\n\t"
        "global_load_dwordx4 %1, %5, off sc1\n\t"
        "global_load_dwordx4 %2, %6, off sc1\n\t"
        "global_load_dwordx4 %3, %7, off sc1\n\t"
        "s_waitcnt vmcnt(0)"
        : "=&v"(t[0]), "=&v"(t[1]), "=&v"(t[2]), "=&v"(t[3])
        : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3])
        : "memory");
  } else if constexpr (N == 2) {
    asm volatile(
        "global_load_dwordx4 %0, %2, off sc1\n\t"
        "global_load_dwordx4 %1, %3, off sc1\n\t"
        "s_waitcnt vmcnt(0)"
        : "=&v"(t[0]), "=&v"(t[1])
        : "v"(p[0]), "v"(p[1])
        : "memory");
  } else {
    asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=&v"(t[0]) : "v"(p[0]) : "memory");
  }
}

// ------------------------------------------------------------------------------------------------
// Per-wave working set handed to a layer for one leapfrog step
// ------------------------------------------------------------------------------------------------
struct StepCtx {
  const float* X;        // this window's rows
  const float* y;
  int n;
  int tile_begin, tile_end;  // 16-row tiles of this wave
  bool x_vec_ok, y_vec_ok;
  const float* ell_prev;  // last step only: rows of the current state (null = zeros)
  float* ell_new;         // last step only: where to store this state's rows (null = skip)
  int* progress;          // LDS, one word per wave: tiles done in this step (null = no balancing)
  int wave, partner;      // this wave and the wave it shares a SIMD with
  float* tile_lds;        // LDS, this wave's copy of the tile it is working on (layers that keep one)
  int back, back_next;    // this gradient evaluation / the next one walks a wave's tiles backwards (layers that
                          // alternate; see leapfrog_walks_back)
};

// Direction of the gradient evaluation of leapfrog step s of L: alternating, and forwards in the last step, so
// that the gradient a chain keeps is always summed in the same order (a chain restored from a saved position
// recomputes it with a one-step launch and must get the same bits).
__device__ __forceinline__ int leapfrog_walks_back(int s, int L) { return (L - 1 - s) & 1; }

// ------------------------------------------------------------------------------------------------
// group barrier: all G workgroups of a chain group have published their partials of this step.
// Bounded: after spin_limit polls, or when another workgroup has given up, the wait ends and the
// launch is abandoned (status[0] set), so every wave always exits.
//
// Everything the workgroups of a group exchange is written with st_agent (write-through to the point
// where all XCDs see it) and read with ld_agent / ld_agent4 (never served from an XCD-local cache
// level), so the barrier needs no L2 write-back and no cache invalidate -- each costs microseconds
// per step and an invalidate would also throw away the cached rows of X.  What it does need is
// ordering: every thread waits until its own stores have been acknowledged (s_waitcnt vmcnt(0))
// before the workgroup signals its arrival, and the exchange loads are issued after the wait.
// Data that is not written with st_agent (per-row log-likelihood terms, chain state, samples) is only
// ever read back by the workgroup that wrote it or after the kernel has ended.
// ------------------------------------------------------------------------------------------------
// bounded poll of a counter by one thread: 1 when it has reached `target`, 0 when the launch is being
// abandoned (another workgroup gave up, or this one has polled spin_limit times)
__device__ __forceinline__ int poll_counter(unsigned* line, unsigned target, unsigned* status,
                                            unsigned spin_limit) {
  unsigned polls = 0;
  while ((int)(__hip_atomic_load(line, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - target) < 0) {
    __builtin_amdgcn_s_sleep(1);
    if ((++polls & 63u) == 0u) {
      if (__hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) return 0;
      if (polls >= spin_limit) {
        __hip_atomic_store(status + 1, (unsigned)blockIdx.x + 1u, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return 0;
      }
    }
  }
  return 1;
}

// ------------------------------------------------------------------------------------------------
// Flagged packets: the exchange of the 22 -> 40 -> 1 kernel needs no barrier.  A value travels as
// 8 bytes {value, flag}, written by one 8-byte store, so it arrives whole; the flag is the number of the
// leapfrog step within the launch (from 1; the host zeroes the exchange area before every launch), and
// a reader polls the packet itself until the flag says it is this step's.  One memory round trip per
// hand-off instead of three (store, counter, load).  Bounded like the barrier: after spin_limit polls,
// or when another workgroup has given up, the reader gives up (status[0] set) and the launch is abandoned.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ void st_packet(unsigned long long* p, float v, unsigned flag) {
  __hip_atomic_store(p, ((unsigned long long)flag << 32) | (unsigned long long)__builtin_bit_cast(unsigned, v),
                     __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned long long ld_packet(const unsigned long long* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// bookkeeping of one more poll; false when the launch is being abandoned
__device__ __forceinline__ bool poll_again(unsigned& polls, unsigned* status, unsigned spin_limit) {
  __builtin_amdgcn_s_sleep(1);
  if ((++polls & 63u) == 0u) {
    if (__hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) return false;
    if (polls >= spin_limit) {
      __hip_atomic_store(status + 1, (unsigned)blockIdx.x + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return false;
    }
  }
  return true;
}
// the value of one packet once its flag is `flag`; `fine` is cleared when the wait is abandoned
__device__ __forceinline__ float wait_packet(const unsigned long long* p, unsigned flag, unsigned* status,
                                             unsigned spin_limit, bool& fine) {
  unsigned polls = 0;
  unsigned long long v = ld_packet(p);
  while ((unsigned)(v >> 32) != flag) {
    if (!poll_again(polls, status, spin_limit)) {
      fine = false;
      break;
    }
    v = ld_packet(p);
  }
  return __builtin_bit_cast(float, (unsigned)v);
}
// (taken by value: applied straight to an element of a vector, __builtin_bit_cast reads element 0)
__device__ __forceinline__ unsigned float_bits(float f) { return __builtin_bit_cast(unsigned, f); }
// Eight 16-byte columns (two packets each) of up to eight records, polled until every packet of the
// first `valid` records carries `flag`.
// N = 1, 2, 4 or 8 loads per poll: only t[0 .. N) and p[0 .. N) are used.
template <int N = 8>
__device__ __forceinline__ void wait_packets4x8(f4 (&t)[8], const unsigned long long* const (&p)[8], int valid,
                                                unsigned flag, unsigned* status, unsigned spin_limit,
                                                bool& fine) {
  const float* q[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) q[k] = reinterpret_cast<const float*>(p[k < N ? k : 0]);
  unsigned polls = 0;
  for (;;) {
    ld_agent4xN<N>(t, q);
    bool ok = true;
#pragma unroll
    for (int k = 0; k < N; ++k)
      if (k < valid)
        ok = ok && float_bits(t[k][1]) == flag && float_bits(t[k][3]) == flag;
    if (ok) break;
    if (!poll_again(polls, status, spin_limit)) {
      fine = false;
      break;
    }
  }
}

// One 16-byte column (two packets), polled until both packets carry `flag`.  Load and wait form one
// assembly statement, as in ld_agent4x8.
__device__ __forceinline__ f4 wait_packets4(const unsigned long long* p, unsigned flag, unsigned* status,
                                            unsigned spin_limit, bool& fine) {
  f4 t;
  unsigned polls = 0;
  for (;;) {
    asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=&v"(t) : "v"(p) : "memory");
    if (float_bits(t[1]) == flag && float_bits(t[3]) == flag) break;
    if (!poll_again(polls, status, spin_limit)) {
      fine = false;
      break;
    }
  }
  return t;
}

// `epoch` counts the barriers of this launch from 1.  Up to 64 workgroups add to the group's counter
// directly.  Larger groups arrive in blocks of 32 ranks at a block counter and the last arriver of a
// block adds to the group's counter: 256 same-address atomics cost 3.8 us, 32 + 8 cost 2.3 us.
// With wait == false the workgroup only announces its arrival (it does not need the others' data).
__device__ __forceinline__ bool group_barrier(unsigned* line, int G, int rank, unsigned epoch,
                                              unsigned* status, unsigned spin_limit, int* s_flag,
                                              bool signal = true, bool wait = true) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this thread's partials have reached memory
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned target;
    if (G <= 64) {
      target = epoch * (unsigned)G;
      if (signal) __hip_atomic_fetch_add(line, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
      const int blk = rank >> 5;
      const unsigned blk_size = (unsigned)min(32, G - 32 * blk);
      target = epoch * (unsigned)((G + 31) >> 5);
      if (signal) {
        const unsigned prev = __hip_atomic_fetch_add(line + 32 * (1 + blk), 1u, __ATOMIC_RELAXED,
                                                     __HIP_MEMORY_SCOPE_AGENT);
        if (prev + 1u == epoch * blk_size)
          __hip_atomic_fetch_add(line, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    *s_flag = wait ? poll_counter(line, target, status, spin_limit) : 1;
  }
  __syncthreads();
  return *s_flag != 0;
}

// Second barrier of the two-phase reduction: only the `n_red` reducing workgroups have something to
// announce (their slice of the totals is stored); everybody waits for all of them.  Uses the last
// nine counter lines of the group.
__device__ __forceinline__ bool reducer_barrier(unsigned* line, int n_red, bool reducer, int rank,
                                                unsigned epoch, unsigned* status, unsigned spin_limit,
                                                int* s_flag, bool signal = true) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (threadIdx.x == 0) {
    // the reducers count themselves on a line nobody polls; the last one releases everybody through
    // eight polled lines (one per block of 32 ranks), each of which sees one atomic per step and 32
    // pollers: polls of one line are served one after the other
    unsigned* arrivals = line + 32 * 9;
    unsigned* release = line + 32 * 10;
    if (reducer && signal) {
      const unsigned prev = __hip_atomic_fetch_add(arrivals, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (prev + 1u == epoch * (unsigned)n_red) {
#pragma unroll
        for (int k = 0; k < 8; ++k)
          __hip_atomic_fetch_add(release + 32 * k, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    *s_flag = poll_counter(release + 32 * ((rank >> 5) & 7), epoch, status, spin_limit);
  }
  __syncthreads();
  return *s_flag != 0;
}

}  // namespace bnn
