// Exponent statistics: per-matrix max exponent, element count above the
// "ignore" threshold and count of elements that would underflow the fp16 lo
// term.  HBM-bound streaming reductions for gfx950: 16-byte loads, wave64
// butterfly reduction, one partial record per workgroup, and the last
// workgroup to arrive folds the partials and takes the mode decision, so a
// statistics pass is a single launch with no zero-initialisation step.
//
// Results are integer counts and a bit-masked maximum, hence independent of the
// reduction order and bit-exact with the reference algorithm
// (src/exp_stats.cu:32-62 counting, :74-184 stage 1 + decision 1, :187-293
// stage 2 + decision 2, :386-459 max only, :295-379 launch arguments).
#include "handle.hpp"
#include "utils.hpp"
#include <cumpsgemm/cumpsgemm.hpp>
#include <cumpsgemm/cumpsgemm_ext.h>
#include <type_traits>

namespace cumpsgemm_amd {
namespace {

// Few, large workgroups: every workgroup ends with one device-scope release
// fence and one ticket atomic, and on a multi-XCD part those cost far more than
// the streaming loop itself when thousands of small workgroups queue up on them.
constexpr int kBlock = 1024;
constexpr int kWaves = kBlock / 64;

struct Acc {
  float mx;
  unsigned total;
  unsigned under;
};

__device__ inline void count_one(Acc &a, float x, float ignore_thr, float under_thr) {
  const float ax = fabsf(x);
  a.mx = fmaxf(a.mx, ax); // NaN operands are ignored
  if (ax >= ignore_thr) {
    a.total++;
    if (ax < under_thr) a.under++;
  }
}

// MODE 0: stage 1 (max + counts, absolute thresholds)
// MODE 1: stage 2 (counts only, thresholds relative to the slot's max exponent;
//                  runs only if the slot is UNDEFINED)
// MODE 2: max exponent only
// One matrix to scan: result slot, scratch for the per-workgroup partials,
// arrival counter, the view of the data and how many workgroups work on it.
struct StatsJob {
  StatsSlot *slot;
  StatsPartial *partials;
  unsigned *ticket;
  const float *ptr;
  unsigned long long count_f; // flat path: number of floats; 0 = strided path
  unsigned m_f, n;
  unsigned long long ld_f;
  unsigned nbatch;
  unsigned long long stride_f;
  unsigned blocks;
};

// A launch scans one matrix or two (A and B of a GEMM: one launch instead of
// two saves a kernel boundary, which costs about as much as scanning 30 MB):
// workgroups [0, job0.blocks) take job0, the rest job1, each job with its own
// partials and arrival counter.
// Ordering of the hand-over from the publishing workgroups to the folding one.
// CUMPSGEMM_STATS_STRICT_ORDER = 1 makes the ticket an acquire-release atomic
// at device scope, which is all the HIP memory model asks for; on gfx950 that
// costs an L2 write-back and invalidate per workgroup, serialised behind one
// another (64 MiB scan: 77 us against 17 us).  The default form relies on three
// properties of gfx950 instead, and refuses to compile for anything else:
//  - an atomic store or load at device scope is performed at the memory side of
//    the fabric (it bypasses the issuing XCD's L2 and the vector L1), so a
//    partial record needs no cache write-back to become visible to another XCD
//    and no invalidate to be read fresh;
//  - s_waitcnt vmcnt(0) / lgkmcnt(0) returns only when those stores have been
//    acknowledged, so every record is in memory before its workgroup's ticket
//    increment is issued;
//  - the compiler keeps relaxed atomics to different addresses in program
//    order around the explicit waitcnt (they are volatile-like memory
//    operations to it).
// A soak test (thousands of launches of every size against an independent
// count) guards the default form.
#ifndef CUMPSGEMM_STATS_STRICT_ORDER
#define CUMPSGEMM_STATS_STRICT_ORDER 0
#endif
#if !CUMPSGEMM_STATS_STRICT_ORDER && defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__)
#error "the fence-free hand-over of exp_stats_kernel is written for gfx950; build with -DCUMPSGEMM_STATS_STRICT_ORDER=1"
#endif
// Stage 2 of a pair can also write the launch flag that the two decisions
// give (flag_out != nullptr; the combination of src/dynamic_scaling.cu:364-385),
// which saves the one-thread kernel that would otherwise follow, i.e. one more
// kernel boundary per AUTO call.  Each job has one finishing thread -- thread 0
// of its first workgroup when stage 1 has already decided and the job's
// workgroups leave at once, thread 0 of its folding workgroup otherwise --
// which takes a ticket of the pair once its job's slot is final; the second of
// the two reads both decisions and writes the flag.  The hand-over between the
// two finishing threads follows the same ordering rules as the partials.
__device__ inline void finish_pair_job(int *flag_out, unsigned *pair_ticket, StatsSlot *slot_a,
                                       StatsSlot *slot_b) {
#if CUMPSGEMM_STATS_STRICT_ORDER
  const unsigned arrived =
      __hip_atomic_fetch_add(pair_ticket, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
#else
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_waitcnt(0);
  const unsigned arrived =
      __hip_atomic_fetch_add(pair_ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#endif
  if (arrived != 1u) return;
  const int pa = __hip_atomic_load(&slot_a->mode, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const int pb = __hip_atomic_load(&slot_b->mode, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  *flag_out = combine_launch_flag(pa, pb);
  __hip_atomic_store(pair_ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int MODE>
__global__ __launch_bounds__(kBlock) void exp_stats_kernel(const StatsJob job0, const StatsJob job1,
                                                           float ignore_thr, float under_thr,
                                                           float tolerance, int *flag_out,
                                                           unsigned *pair_ticket) {
  const bool second = blockIdx.x >= job0.blocks; // uniform
  const StatsJob &job = second ? job1 : job0;
  StatsSlot *const slot = job.slot;
  StatsPartial *const partials = job.partials;
  unsigned *const ticket = job.ticket;
  const float *const ptr = job.ptr;
  const unsigned long long count_f = job.count_f, ld_f = job.ld_f, stride_f = job.stride_f;
  const unsigned m_f = job.m_f, n = job.n, nbatch = job.nbatch;
  const unsigned nblocks = job.blocks, bid = blockIdx.x - (second ? job0.blocks : 0u);
  if (MODE == 1) {
    if (slot->mode != CUMPSGEMM_UNDEFINED) { // uniform across the job's workgroups
      if (flag_out != nullptr && bid == 0 && threadIdx.x == 0)
        finish_pair_job(flag_out, pair_ticket, job0.slot, job1.slot);
      return;
    }
    const float max_exp = __uint_as_float(slot->max_exp_bits);
    ignore_thr *= max_exp;
    under_thr *= max_exp;
  }
  Acc acc{0.0f, 0u, 0u};
  const unsigned tid = threadIdx.x;
  if (count_f != 0) {
    // contiguous data: head up to 16-byte alignment, float4 body, tail
    const unsigned long long mis = ((16 - ((uintptr_t)ptr & 15)) & 15) / 4;
    const unsigned long long head = mis < count_f ? mis : count_f;
    const float4 *body = reinterpret_cast<const float4 *>(ptr + head);
    const unsigned long long nvec = (count_f - head) / 4;
    const unsigned long long gsz = (unsigned long long)nblocks * kBlock;
    unsigned long long i = (unsigned long long)bid * kBlock + tid;
    auto count4 = [&](const float4 &v) {
      count_one(acc, v.x, ignore_thr, under_thr); count_one(acc, v.y, ignore_thr, under_thr);
      count_one(acc, v.z, ignore_thr, under_thr); count_one(acc, v.w, ignore_thr, under_thr);
    };
    // Eight independent 16-byte loads in flight per thread.  A workgroup takes
    // contiguous chunks of 8 * kBlock vectors, so that what the whole grid
    // streams at any moment is one compact window (windows a power-of-two
    // stride apart would fall on the same memory channels).
    constexpr unsigned long long kChunk = 8ull * kBlock;
    const unsigned long long nfull = nvec / kChunk;
    for (unsigned long long c = bid; c < nfull; c += nblocks) {
      const float4 *cp = body + c * kChunk + tid;
      float4 v[8];
#pragma unroll
      for (int j = 0; j < 8; j++) v[j] = cp[j * kBlock];
#pragma unroll
      for (int j = 0; j < 8; j++) count4(v[j]);
    }
    i += nfull * kChunk;
    for (; i < nvec; i += gsz) {
      count4(body[i]);
    }
    if (bid == 0) {
      if (tid < head) count_one(acc, ptr[tid], ignore_thr, under_thr);
      const unsigned long long tail0 = head + nvec * 4;
      if (tail0 + tid < count_f) count_one(acc, ptr[tail0 + tid], ignore_thr, under_thr);
    }
  } else {
    // strided view: one column (of m_f floats) per wave iteration
    const unsigned long long ncols = (unsigned long long)n * nbatch;
    const unsigned lane = tid & 63;
    for (unsigned long long col = (unsigned long long)bid * kWaves + (tid >> 6); col < ncols;
         col += (unsigned long long)nblocks * kWaves) {
      const float *cp = ptr + (col / n) * stride_f + (col % n) * ld_f;
      unsigned i = lane;
      for (; i + 192 < m_f; i += 256) {
        const float x0 = cp[i], x1 = cp[i + 64], x2 = cp[i + 128], x3 = cp[i + 192];
        count_one(acc, x0, ignore_thr, under_thr); count_one(acc, x1, ignore_thr, under_thr);
        count_one(acc, x2, ignore_thr, under_thr); count_one(acc, x3, ignore_thr, under_thr);
      }
      for (; i < m_f; i += 64) count_one(acc, cp[i], ignore_thr, under_thr);
    }
  }

  // wave64 butterfly
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    acc.mx = fmaxf(acc.mx, __shfl_xor(acc.mx, off, 64));
    acc.total += __shfl_xor(acc.total, off, 64);
    acc.under += __shfl_xor(acc.under, off, 64);
  }
  __shared__ float s_mx[kBlock / 64];
  __shared__ unsigned s_total[kBlock / 64], s_under[kBlock / 64];
  __shared__ bool s_last;
  if ((tid & 63) == 0) {
    s_mx[tid >> 6] = acc.mx;
    s_total[tid >> 6] = acc.total;
    s_under[tid >> 6] = acc.under;
  }
  __syncthreads();
  if (tid < 64) {
    // first wave: fold the per-wave results with a second butterfly
    float mx = tid < kWaves ? s_mx[tid] : 0.0f;
    unsigned long long t = tid < kWaves ? s_total[tid] : 0ull;
    unsigned long long u = tid < kWaves ? s_under[tid] : 0ull;
#pragma unroll
    for (int off = kWaves / 2; off >= 1; off >>= 1) {
      mx = fmaxf(mx, __shfl_xor(mx, off, 64));
      t += __shfl_xor(t, off, 64);
      u += __shfl_xor(u, off, 64);
    }
    if (tid == 0) {
      // Publish the partial record with device-scope (write-through) stores, wait
      // for them to be acknowledged, then take a ticket.  A device-scope release
      // fence here instead would write back the whole L2 once per workgroup, and
      // those write-backs serialise: they cost several times the streaming loop.
      StatsPartial *p = partials + bid;
      __hip_atomic_store(&p->max_bits, __float_as_uint(mx) & 0x7f800000u, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(&p->total, t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(&p->underflow, u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#if CUMPSGEMM_STATS_STRICT_ORDER
      // the portable form: the ticket is a release / acquire operation at device scope
      const unsigned arrived =
          __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
#else
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __builtin_amdgcn_s_waitcnt(0);
      const unsigned arrived =
          __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#endif
      s_last = (arrived == nblocks - 1);
    }
  }
  __syncthreads();
  if (!s_last) return;

  // last workgroup: fold all partials (device-scope loads, independent of each
  // other so that they are all in flight together).  No fence is needed: every
  // partial was acknowledged by memory before its workgroup took a ticket, the
  // last ticket was taken before the barrier above, and device-scope loads do
  // not look at this XCD's L2.
  unsigned mxb = 0;
  unsigned long long t = 0, u = 0;
  for (unsigned i = tid; i < nblocks; i += kBlock) {
    StatsPartial *p = partials + i;
    const unsigned b = __hip_atomic_load(&p->max_bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned long long pt = __hip_atomic_load(&p->total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned long long pu = __hip_atomic_load(&p->underflow, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    mxb = b > mxb ? b : mxb;
    t += pt;
    u += pu;
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const unsigned ob = __shfl_xor(mxb, off, 64);
    mxb = ob > mxb ? ob : mxb;
    t += __shfl_xor(t, off, 64);
    u += __shfl_xor(u, off, 64);
  }
  __shared__ unsigned r_mx[kBlock / 64];
  __shared__ unsigned long long r_t[kBlock / 64], r_u[kBlock / 64];
  if ((tid & 63) == 0) {
    r_mx[tid >> 6] = mxb;
    r_t[tid >> 6] = t;
    r_u[tid >> 6] = u;
  }
  __syncthreads();
  if (tid >= 64) return;
  mxb = tid < kWaves ? r_mx[tid] : 0u;
  t = tid < kWaves ? r_t[tid] : 0ull;
  u = tid < kWaves ? r_u[tid] : 0ull;
#pragma unroll
  for (int off = kWaves / 2; off >= 1; off >>= 1) {
    const unsigned ob = __shfl_xor(mxb, off, 64);
    mxb = ob > mxb ? ob : mxb;
    t += __shfl_xor(t, off, 64);
    u += __shfl_xor(u, off, 64);
  }
  if (tid == 0) {
    if (MODE == 0) {
      slot->max_exp_bits = mxb;
      const float max_exp = __uint_as_float(mxb);
      // decision 1: counters compared as floats, like the reference's mixed
      // u64 * float expression
      if (((float)u > (float)t * tolerance) || (max_exp > 0.0f && t == 0)) {
        slot->mode = CUMPSGEMM_UNDEFINED;
        slot->total = 0;
        slot->underflow = 0;
      } else {
        slot->mode = CUMPSGEMM_FP16TCEC;
        slot->total = t;
        slot->underflow = u;
      }
    } else if (MODE == 1) {
      slot->total = t;
      slot->underflow = u;
      const int decided = ((float)u <= (float)t * tolerance) ? CUMPSGEMM_FP16TCEC_SCALING
                                                             : CUMPSGEMM_TF32TCEC;
      // (a device-scope store: the other job's finishing thread may read it in this launch)
      __hip_atomic_store(&slot->mode, decided, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
      slot->max_exp_bits = mxb;
    }
    // ready for the next pass on this stream
    // (the slot and the ticket become visible to later kernels at the end of this one)
    __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (MODE == 1 && flag_out != nullptr) finish_pair_job(flag_out, pair_ticket, job0.slot, job1.slot);
  }
}

struct View {
  unsigned long long count_f; // != 0 -> contiguous
  unsigned m_f, n, nbatch;
  unsigned long long ld_f, stride_f;
  unsigned grid;
};

template <class T>
View make_view(const cuMpSGEMM_handle *h, unsigned m, unsigned n, unsigned ld, unsigned batch,
               unsigned stride) {
  constexpr unsigned ES = std::is_same<T, hipComplex>::value ? 2 : 1;
  View v{};
  // stride == 0 -> only the first matrix is looked at (reference src/exp_stats.cu:306)
  v.nbatch = (stride == 0) ? 1 : batch;
  v.m_f = m * ES;
  v.n = n;
  v.ld_f = (unsigned long long)ld * ES;
  v.stride_f = (unsigned long long)stride * ES;
  const bool dense_cols = (ld == m) || n == 1;
  const bool dense_batch = v.nbatch == 1 || (unsigned long long)stride == (unsigned long long)m * n;
  const unsigned long long total_f = (unsigned long long)m * n * v.nbatch * ES;
  unsigned long long blocks;
  if (dense_cols && dense_batch) {
    v.count_f = total_f;
    blocks = (total_f / 4 + kBlock * 4 - 1) / (kBlock * 4);
  } else {
    v.count_f = 0;
    blocks = ((unsigned long long)n * v.nbatch + kWaves - 1) / kWaves;
  }
  // one 16-wave workgroup per CU streams at full HBM rate; more workgroups only
  // lengthen the serial ticket chain at the end
  const unsigned long long cap = std::min<unsigned long long>((unsigned long long)h->num_cus, kMaxStatsBlocks);
  v.grid = (unsigned)std::max<unsigned long long>(1, std::min(blocks, cap));
  return v;
}

unsigned next_slot(cuMpSGEMM_handle *h) {
  // ring of result slots: 0 and 1 are presets, 2..length-1 cycle
  // (reference src/exp_stats.cu:15-24)
  h->stats_current_id++;
  if (h->stats_current_id >= h->stats_ring_length) h->stats_current_id = 2;
  return h->stats_current_id;
}

template <class T>
StatsJob make_job(cuMpSGEMM_handle *h, const View &v, const T *ptr, unsigned slot_id, unsigned which,
                  unsigned first_partial) {
  StatsJob j{};
  j.slot = h->stats_slots + slot_id;
  j.partials = h->stats_partials + first_partial;
  j.ticket = h->stats_ticket + which;
  j.ptr = reinterpret_cast<const float *>(ptr);
  j.count_f = v.count_f;
  j.m_f = v.m_f;
  j.n = v.n;
  j.ld_f = v.ld_f;
  j.nbatch = v.nbatch;
  j.stride_f = v.stride_f;
  j.blocks = v.grid;
  return j;
}

// MODE 0 + 1 (full statistics) or 2 (maximum only) over one job or two
template <bool FULL>
void launch_stats(cuMpSGEMM_handle *h, const StatsJob &j0, const StatsJob &j1, int *flag_out = nullptr) {
  // (a null matrix would fault on the device; an empty one has nothing to read)
  const bool bad0 = j0.ptr == nullptr && j0.m_f != 0 && j0.n != 0;
  const bool bad1 = j1.blocks != 0 && j1.ptr == nullptr && j1.m_f != 0 && j1.n != 0;
  if (bad0 || bad1) {
    log_error("exponent statistics: null matrix pointer, nothing scanned");
    return;
  }
  const dim3 grid(j0.blocks + j1.blocks);
  if (FULL) {
    {
      ProfileScope prof(h, "exp_stats_1");
      hipLaunchKernelGGL(exp_stats_kernel<0>, grid, dim3(kBlock), 0, h->stream, j0, j1, h->ignore_threshold,
                         h->underflow_threshold, h->underflow_tolerance_rate, (int *)nullptr,
                         (unsigned *)nullptr);
    }
    {
      ProfileScope prof(h, "exp_stats_2");
      // stage-2 thresholds are half the stage-1 ones, times the max exponent
      // (reference src/exp_stats.cu:360-361, :205-206)
      // (the launch flag of a pair is written by this launch when the caller asks for it)
      const bool with_flag = flag_out != nullptr && j0.blocks != 0 && j1.blocks != 0;
      hipLaunchKernelGGL(exp_stats_kernel<1>, grid, dim3(kBlock), 0, h->stream, j0, j1, h->ignore_threshold / 2,
                         h->underflow_threshold / 2, h->underflow_tolerance_rate,
                         with_flag ? flag_out : (int *)nullptr, h->stats_ticket + 2);
    }
  } else {
    ProfileScope prof(h, "exp_max");
    hipLaunchKernelGGL(exp_stats_kernel<2>, grid, dim3(kBlock), 0, h->stream, j0, j1, 0.0f, 0.0f, 0.0f,
                       (int *)nullptr, (unsigned *)nullptr);
  }
}

template <class T>
void run_exp_stats(cuMpSGEMM_handle *h, unsigned m, unsigned n, const T *ptr, unsigned ld,
                   unsigned batch, unsigned stride, unsigned slot_id) {
  const View v = make_view<T>(h, m, n, ld, batch, stride);
  launch_stats<true>(h, make_job<T>(h, v, ptr, slot_id, 0, 0), StatsJob{});
}

template <class T>
void run_exp_max(cuMpSGEMM_handle *h, unsigned m, unsigned n, const T *ptr, unsigned ld,
                 unsigned batch, unsigned stride, unsigned slot_id) {
  const View v = make_view<T>(h, m, n, ld, batch, stride);
  launch_stats<false>(h, make_job<T>(h, v, ptr, slot_id, 0, 0), StatsJob{});
}

// Two matrices in one launch; the workgroups (one per CU) are shared out in
// proportion to the sizes.
template <class T, bool FULL>
void run_pair(cuMpSGEMM_handle *h, const MatrixView<T> &a, unsigned slot_a, const MatrixView<T> &b,
              unsigned slot_b, int *flag_out = nullptr) {
  View va = make_view<T>(h, a.m, a.n, a.ld, a.batch, a.stride);
  View vb = make_view<T>(h, b.m, b.n, b.ld, b.batch, b.stride);
  const unsigned long long cap = std::min<unsigned long long>((unsigned long long)h->num_cus, kMaxStatsBlocks);
  if ((unsigned long long)va.grid + vb.grid > cap) {
    const double wa = (double)a.m * a.n * va.nbatch, wb = (double)b.m * b.n * vb.nbatch;
    unsigned ga = (unsigned)((double)cap * wa / (wa + wb) + 0.5);
    ga = std::max(1u, std::min(ga, (unsigned)cap - 1u));
    va.grid = std::min(va.grid, ga);
    vb.grid = std::min(vb.grid, (unsigned)cap - va.grid);
  }
  launch_stats<FULL>(h, make_job<T>(h, va, a.ptr, slot_a, 0, 0), make_job<T>(h, vb, b.ptr, slot_b, 1, va.grid),
                     flag_out);
}

void read_slot(cuMpSGEMM_handle *h, unsigned id, StatsSlot &out) {
  check_hip(hipMemcpyAsync(&out, h->stats_slots + id, sizeof(StatsSlot), hipMemcpyDeviceToHost,
                           h->stream),
            "read stats slot");
  check_hip(hipStreamSynchronize(h->stream), "sync after stats read");
}
} // namespace

template <class T>
void exp_stats_pair(cuMpSGEMM_handle *h, const MatrixView<T> &a, const MatrixView<T> &b, unsigned &a_id,
                    unsigned &b_id, int flag_id) {
  a_id = next_slot(h);
  b_id = next_slot(h);
  run_pair<T, true>(h, a, a_id, b, b_id, flag_id >= 0 ? h->flag_buffer + flag_id : nullptr);
}
template <class T>
void exp_max_pair(cuMpSGEMM_handle *h, const MatrixView<T> &a, const MatrixView<T> &b, unsigned &a_id,
                  unsigned &b_id) {
  a_id = next_slot(h);
  b_id = next_slot(h);
  run_pair<T, false>(h, a, a_id, b, b_id);
}
template void exp_stats_pair<float>(cuMpSGEMM_handle *, const MatrixView<float> &, const MatrixView<float> &,
                                    unsigned &, unsigned &, int);
template void exp_stats_pair<hipComplex>(cuMpSGEMM_handle *, const MatrixView<hipComplex> &,
                                         const MatrixView<hipComplex> &, unsigned &, unsigned &, int);
template void exp_max_pair<float>(cuMpSGEMM_handle *, const MatrixView<float> &, const MatrixView<float> &,
                                  unsigned &, unsigned &);
template void exp_max_pair<hipComplex>(cuMpSGEMM_handle *, const MatrixView<hipComplex> &,
                                       const MatrixView<hipComplex> &, unsigned &, unsigned &);
} // namespace cumpsgemm_amd

using namespace cumpsgemm_amd;

template <class T>
unsigned cumpsgemm::exp_stats_ext(handle_t handle, unsigned m, unsigned n, const T *ptr,
                                  unsigned ld, unsigned batch_size, unsigned stride) {
  const unsigned id = next_slot(handle);
  run_exp_stats<T>(handle, m, n, ptr, ld, batch_size, stride, id);
  return id;
}
template <class T>
unsigned cumpsgemm::exp_max_ext(handle_t handle, unsigned m, unsigned n, const T *ptr,
                                unsigned ld, unsigned batch_size, unsigned stride) {
  const unsigned id = next_slot(handle);
  run_exp_max<T>(handle, m, n, ptr, ld, batch_size, stride, id);
  return id;
}
template unsigned cumpsgemm::exp_stats_ext<float>(handle_t, unsigned, unsigned, const float *,
                                                  unsigned, unsigned, unsigned);
template unsigned cumpsgemm::exp_stats_ext<hipComplex>(handle_t, unsigned, unsigned,
                                                       const hipComplex *, unsigned, unsigned,
                                                       unsigned);
template unsigned cumpsgemm::exp_max_ext<float>(handle_t, unsigned, unsigned, const float *,
                                                unsigned, unsigned, unsigned);
template unsigned cumpsgemm::exp_max_ext<hipComplex>(handle_t, unsigned, unsigned,
                                                     const hipComplex *, unsigned, unsigned,
                                                     unsigned);

std::pair<std::size_t, std::size_t> cumpsgemm::get_exp_stats(handle_t handle, unsigned buffer_id) {
  StatsSlot s;
  read_slot(handle, buffer_id, s);
  return {(std::size_t)s.underflow, (std::size_t)s.total}; // reference src/exp_stats.cu:628
}
unsigned cumpsgemm::get_current_exp_stats_buffer_id(handle_t handle) {
  return handle->stats_current_id;
}
void cumpsgemm::reset_exp_stats_buffer_id(handle_t handle) { handle->stats_current_id = 1; }
void cumpsgemm::set_exp_stats_params(handle_t handle, float ignore_threshold,
                                     float underflow_threshold, float underflow_ratio_tolerance) {
  handle->ignore_threshold = ignore_threshold;
  handle->underflow_threshold = underflow_threshold;
  handle->underflow_tolerance_rate = underflow_ratio_tolerance;
}
void cumpsgemm::enable_exp_stats(handle_t handle) { handle->exp_stats_enabled = true; }
void cumpsgemm::disable_exp_stats(handle_t handle) { handle->exp_stats_enabled = false; }
float cumpsgemm::get_max_exp(handle_t handle, unsigned buffer_id) {
  StatsSlot s;
  read_slot(handle, buffer_id, s);
  float f;
  static_assert(sizeof(f) == sizeof(s.max_exp_bits), "");
  std::memcpy(&f, &s.max_exp_bits, sizeof(f));
  return f;
}
cuMpSGEMM_compute_mode_t cumpsgemm::get_exp_stats_compute_mode_level(handle_t handle,
                                                                     unsigned buffer_id) {
  StatsSlot s;
  read_slot(handle, buffer_id, s);
  return (cuMpSGEMM_compute_mode_t)s.mode;
}

void cumpsgemm::enable_exp_stats_profiling(handle_t handle) { handle->profiler.enabled = true; }
void cumpsgemm::disable_exp_stats_profiling(handle_t handle) { handle->profiler.enabled = false; }
void cumpsgemm::reset_exp_stats_profiling(handle_t handle) { handle->profiler.entries.clear(); }
void cumpsgemm::print_exp_stats_profiling(handle_t handle, unsigned csv) {
  double total = 0.0;
  for (const auto &e : handle->profiler.entries) total += e.second.sum;
  if (csv) {
    std::printf("name,sum_s,n,avg_s,ratio\n");
    for (const auto &e : handle->profiler.entries)
      std::printf("%s,%e,%llu,%e,%e\n", e.first.c_str(), e.second.sum,
                  (unsigned long long)e.second.n, e.second.sum / e.second.n,
                  total > 0 ? e.second.sum / total : 0.0);
  } else {
    for (const auto &e : handle->profiler.entries)
      std::printf("%20s : %e [s] (%6.2f%%), n = %llu, avg = %e [s]\n", e.first.c_str(),
                  e.second.sum, total > 0 ? 100.0 * e.second.sum / total : 0.0,
                  (unsigned long long)e.second.n, e.second.sum / e.second.n);
  }
  std::fflush(stdout);
}
std::unordered_map<std::string, cumpsgemm::debug::stats_t>
cumpsgemm::debug::get_exp_stats_profiling_result(handle_t handle) {
  std::unordered_map<std::string, stats_t> r;
  for (const auto &e : handle->profiler.entries) r[e.first] = stats_t{e.second.sum, e.second.n};
  return r;
}

extern "C" {
unsigned cuMpSGEMM_exp_stats_ext_s(cuMpSGEMM_handle_t h, unsigned m, unsigned n, const float *ptr,
                                   unsigned ld, unsigned batch, unsigned stride) {
  return cumpsgemm::exp_stats_ext<float>(h, m, n, ptr, ld, batch, stride);
}
unsigned cuMpSGEMM_exp_stats_ext_c(cuMpSGEMM_handle_t h, unsigned m, unsigned n,
                                   const hipComplex *ptr, unsigned ld, unsigned batch,
                                   unsigned stride) {
  return cumpsgemm::exp_stats_ext<hipComplex>(h, m, n, ptr, ld, batch, stride);
}
unsigned cuMpSGEMM_exp_max_ext_s(cuMpSGEMM_handle_t h, unsigned m, unsigned n, const float *ptr,
                                 unsigned ld, unsigned batch, unsigned stride) {
  return cumpsgemm::exp_max_ext<float>(h, m, n, ptr, ld, batch, stride);
}
unsigned cuMpSGEMM_exp_max_ext_c(cuMpSGEMM_handle_t h, unsigned m, unsigned n,
                                 const hipComplex *ptr, unsigned ld, unsigned batch,
                                 unsigned stride) {
  return cumpsgemm::exp_max_ext<hipComplex>(h, m, n, ptr, ld, batch, stride);
}
void cuMpSGEMM_exp_stats_pair_s(cuMpSGEMM_handle_t h, unsigned m_a, unsigned n_a, const float *a,
                                unsigned lda, unsigned m_b, unsigned n_b, const float *b,
                                unsigned ldb, int flag_id, unsigned *ids_out) {
  unsigned ia = 0, ib = 0;
  exp_stats_pair<float>(h, MatrixView<float>{a, m_a, n_a, lda, 1u, 0u}, MatrixView<float>{b, m_b, n_b, ldb, 1u, 0u},
                        ia, ib, flag_id);
  if (ids_out != nullptr) {
    ids_out[0] = ia;
    ids_out[1] = ib;
  }
}
void cuMpSGEMM_exp_max_pair_s(cuMpSGEMM_handle_t h, unsigned m_a, unsigned n_a, const float *a,
                              unsigned lda, unsigned m_b, unsigned n_b, const float *b,
                              unsigned ldb, unsigned *ids_out) {
  unsigned ia = 0, ib = 0;
  exp_max_pair<float>(h, MatrixView<float>{a, m_a, n_a, lda, 1u, 0u}, MatrixView<float>{b, m_b, n_b, ldb, 1u, 0u},
                      ia, ib);
  if (ids_out != nullptr) {
    ids_out[0] = ia;
    ids_out[1] = ib;
  }
}
// The read-backs synchronise the stream and the C++ forms throw when HIP
// reports an error; no exception may cross the C boundary, so the C forms log
// (check_hip already has) and return zeros / UNDEFINED instead.
void cuMpSGEMM_get_exp_stats(cuMpSGEMM_handle_t h, unsigned id, uint64_t *underflow,
                             uint64_t *total) {
  *underflow = 0;
  *total = 0;
  try {
    const auto r = cumpsgemm::get_exp_stats(h, id);
    *underflow = r.first;
    *total = r.second;
  } catch (const std::exception &) {
  }
}
float cuMpSGEMM_get_max_exp(cuMpSGEMM_handle_t h, unsigned id) {
  try {
    return cumpsgemm::get_max_exp(h, id);
  } catch (const std::exception &) {
    return 0.0f;
  }
}
int cuMpSGEMM_get_exp_stats_compute_mode_level(cuMpSGEMM_handle_t h, unsigned id) {
  try {
    return (int)cumpsgemm::get_exp_stats_compute_mode_level(h, id);
  } catch (const std::exception &) {
    return (int)CUMPSGEMM_UNDEFINED;
  }
}
void cuMpSGEMM_set_exp_stats_params(cuMpSGEMM_handle_t h, float ignore_threshold,
                                    float underflow_threshold, float tolerance) {
  cumpsgemm::set_exp_stats_params(h, ignore_threshold, underflow_threshold, tolerance);
}
unsigned cuMpSGEMM_get_current_exp_stats_buffer_id(cuMpSGEMM_handle_t h) {
  return cumpsgemm::get_current_exp_stats_buffer_id(h);
}
void cuMpSGEMM_reset_exp_stats_buffer_id(cuMpSGEMM_handle_t h) {
  cumpsgemm::reset_exp_stats_buffer_id(h);
}
void cuMpSGEMM_enable_exp_stats(cuMpSGEMM_handle_t h) { cumpsgemm::enable_exp_stats(h); }
void cuMpSGEMM_disable_exp_stats(cuMpSGEMM_handle_t h) { cumpsgemm::disable_exp_stats(h); }
void cuMpSGEMM_enable_exp_stats_profiling(cuMpSGEMM_handle_t h) {
  cumpsgemm::enable_exp_stats_profiling(h);
}
void cuMpSGEMM_disable_exp_stats_profiling(cuMpSGEMM_handle_t h) {
  cumpsgemm::disable_exp_stats_profiling(h);
}
void cuMpSGEMM_reset_exp_stats_profiling(cuMpSGEMM_handle_t h) {
  cumpsgemm::reset_exp_stats_profiling(h);
}
void cuMpSGEMM_print_exp_stats_profiling(cuMpSGEMM_handle_t h, unsigned csv) {
  cumpsgemm::print_exp_stats_profiling(h, csv);
}
int cuMpSGEMM_get_exp_stats_profiling_entry(cuMpSGEMM_handle_t h, const char *name,
                                            double *time_sum, uint64_t *n) {
  if (!h || !name) return 0;
  const auto it = h->profiler.entries.find(name);
  if (it == h->profiler.entries.end()) return 0;
  if (time_sum) *time_sum = it->second.sum;
  if (n) *n = it->second.n;
  return 1;
}
} // extern "C"
