// K5: TeaCache relative-L1 reduction. One streaming read of `cur` and `prev`
// (algorithmic traffic 2 * B*n * sizeof(T)), per-batch-row sums, ONE launch, fixed reduction tree:
//   grid (nblk, B): every workgroup reduces one contiguous slice of one row to two fp32 partials, stores
//   them, and takes a ticket from the row's counter; the workgroup that draws the row's last ticket adds
//   the row's nblk partials in fp64, in slot order, and writes sums[b] = {sum|cur-prev|, sum|prev|}.
// Which workgroup comes last depends on timing, what it computes does not: the tree depends only on
// (B, n), so repeated calls give bit-identical sums.
//
// Scratch layout: a counter region of fixed size (one 64-bit ticket word per row, room for the largest row
// count the entry point accepts, so that no byte of it is ever used for anything else), then the partials
// (B * nblk float pairs). A ticket word is (epoch << 16 | tickets drawn): every launch has an epoch larger
// than any earlier one of the process, a workgroup first raises its row's word to (epoch << 16) with an
// atomic maximum and then draws its ticket with an atomic add, so whatever an earlier launch left in the
// word (one that never finished, say) is overridden. The last workgroup of a row puts the word back to zero
// (a launch replayed from a HIP graph carries the same epoch every time). The region only has to be zero
// ONCE, when the scratch is allocated.
#include "odit_common.h"

#include <mutex>

namespace odit {

constexpr int kRelL1MaxBlocksPerRow = 256;
constexpr int kRelL1VecsPerThread = 4;
// Measured at B = 2, n = 12.6 M bf16 (100 MB): 256 workgroups of 1024 threads 21.9 us; 512 x 512 22.4; 1024 x 256
// 25.9; 3072 x 256 45 us: the tickets are device-scope atomics on one address per row and serialise at ~25 ns each.
constexpr int kRelL1Threads = 1024;     // threads per workgroup
constexpr int kRelL1TotalBlocks = 256;  // workgroups of a launch, over all rows (when rows are long enough)
constexpr int kRelL1MaxRows = 65535;  // grid.y limit
// rows of the no-allocation entry point, whose scratch is a fixed array in device memory
constexpr int kRelL1StaticRows = 64;

// counter region of a caller's workspace: one word for each of the kRelL1MaxRows rows a call may have,
// whatever B a particular call has (a region sized by B would let one call's partials be a later call's
// counters)
constexpr size_t kRelL1RowWordBytes = (static_cast<size_t>(kRelL1MaxRows) + 1) * sizeof(uint64_t);
// Behind the rows' words, group words: a row of more than kRelL1GroupAbove workgroups (few, long rows) draws its
// tickets in two levels, workgroup x from the word of group x % kRelL1Groups and only each group's last arrival
// from the row's word. Atomics on one address are applied one after the other (~20 ns each, and every workgroup
// arrives within the kernel's last microsecond). Measured for 2 x 12.6 M bf16 elements on one box: two atomics per
// workgroup on the row's word at the end of the kernel 24.7 us; the first of them moved to the start of the kernel
// 23.0; 16 arrivals per group word and 8 on the row's word 21.6; one atomic per workgroup and nothing to override
// stale words with 20.0; no tickets and no final sum at all 19.2. Group words are 1 KiB apart so that they sit in
// different memory channels.
constexpr int kRelL1Groups = 8;
constexpr int kRelL1GroupAbove = 32;
constexpr int kRelL1GroupedRows = kRelL1TotalBlocks / (kRelL1GroupAbove + 1);  // rows that can have that many workgroups
constexpr int kRelL1GroupStrideWords = 128;
constexpr size_t kRelL1GroupBytes =
    static_cast<size_t>(kRelL1GroupedRows) * kRelL1Groups * kRelL1GroupStrideWords * sizeof(uint64_t);
constexpr size_t kRelL1CounterBytes = kRelL1RowWordBytes + kRelL1GroupBytes;

static inline int rel_l1_blocks_per_row(int B, int64_t n) {
  // at least one pass of four 16-byte vectors per thread (sized on 8-element vectors; fp32 rows get twice the
  // vectors), at most kRelL1TotalBlocks workgroups over all rows: every workgroup ends with one device-scope
  // atomic on its row's counter, and those serialise
  const int64_t per_block = static_cast<int64_t>(kRelL1Threads) * kRelL1VecsPerThread * 8;
  int64_t nb = (n + per_block - 1) / per_block;
  int64_t cap = kRelL1TotalBlocks / (B > 0 ? B : 1);
  if (cap < 1) cap = 1;
  if (cap > kRelL1MaxBlocksPerRow) cap = kRelL1MaxBlocksPerRow;
  if (nb > cap) nb = cap;
  if (nb < 1) nb = 1;
  return static_cast<int>(nb);
}

template <typename T, bool REF_ROUND>
__global__ __launch_bounds__(kRelL1Threads) void rel_l1_kernel(const T* __restrict__ cur, const T* __restrict__ prev,
                                                     float* partials, uint64_t* counters, uint64_t* groups, uint64_t epoch,
                                                     double* __restrict__ sums, int64_t n, int64_t n_vec,
                                                     int64_t cur_stride, int64_t prev_stride) {
  constexpr int EPV = Vec16<T>::N;
  const int b = blockIdx.y;
  const int nblk = gridDim.x;
  const T* c = cur + b * cur_stride;
  const T* p = prev + b * prev_stride;
  // contiguous slice of vectors for this block
  const int64_t per_blk = (n_vec + nblk - 1) / nblk;
  const int64_t v_begin = static_cast<int64_t>(blockIdx.x) * per_blk;
  const int64_t v_end = v_begin + per_blk < n_vec ? v_begin + per_blk : n_vec;
  // Two-level tickets for rows of many workgroups (groups == nullptr: one level always)
  const bool grouped = groups != nullptr && nblk > kRelL1GroupAbove && b < kRelL1GroupedRows;
  const int grp = static_cast<int>(blockIdx.x) % kRelL1Groups;
  uint64_t* const my_word = grouped ? groups + (static_cast<int64_t>(b) * kRelL1Groups + grp) * kRelL1GroupStrideWords : counters + b;
  const uint64_t my_arrivals = grouped ? static_cast<uint64_t>((nblk - grp + kRelL1Groups - 1) / kRelL1Groups) : static_cast<uint64_t>(nblk);
  // The word this workgroup draws from is raised to the launch's epoch here, long before the tickets are drawn (a
  // no-op for all but the word's first arrival; no value comes back, nothing waits for it): at the end of the
  // kernel each workgroup then waits for one atomic, not two.
  const uint64_t base = epoch << 16;
  if (threadIdx.x == 0) __hip_atomic_fetch_max(my_word, base, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  float sd = 0.f, sp = 0.f;
  auto accumulate = [&](const Vec16<T>& cv, const Vec16<T>& pv) {
#pragma unroll
    for (int j = 0; j < EPV; ++j) {
      const float pf = to_float(pv.e[j]);
      float d = to_float(cv.e[j]) - pf;
      if (REF_ROUND) d = round_to<T>(d);
      sd += fabsf(d);
      sp += fabsf(pf);
    }
  };
  // four vector pairs (eight 16-byte loads) in flight per lane before the first use
  constexpr int U = 4;
  int64_t i = v_begin + threadIdx.x;
  constexpr int NT = kRelL1Threads;
  for (; i + (U - 1) * NT < v_end; i += U * NT) {
    Vec16<T> cv[U], pv[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      cv[u] = load16_stream(c + (i + u * NT) * EPV);
      pv[u] = load16_stream(p + (i + u * NT) * EPV);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) accumulate(cv[u], pv[u]);
  }
  for (; i < v_end; i += NT) accumulate(load16_stream(c + i * EPV), load16_stream(p + i * EPV));
  if (blockIdx.x == 0) {  // scalar tail (also the whole row when vector loads are not possible)
    for (int64_t i = n_vec * EPV + threadIdx.x; i < n; i += NT) {
      const float pf = to_float(p[i]);
      float d = to_float(c[i]) - pf;
      if (REF_ROUND) d = round_to<T>(d);
      sd += fabsf(d);
      sp += fabsf(pf);
    }
  }
  sd = wave_sum(sd);
  sp = wave_sum(sp);
  constexpr int NWAVE = kRelL1Threads / 64;
  __shared__ float red[2][NWAVE];
  __shared__ bool last_of_row;
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) { red[0][wave] = sd; red[1][wave] = sp; }
  __syncthreads();
  if (threadIdx.x == 0) {
    float* out = partials + (static_cast<int64_t>(b) * nblk + blockIdx.x) * 2;
    float o0 = 0.f, o1 = 0.f;
#pragma unroll
    for (int w = 0; w < NWAVE; ++w) { o0 += red[0][w]; o1 += red[1][w]; }   // fixed order
    // The partials go out as device-scope stores (written through to memory, past the XCD-private L2), the wait
    // lets them land, then the ticket is drawn: the last workgroup's device-scope loads below see every partial
    // of the row. A release/acquire pair on the ticket would do the same through a write-back and an
    // invalidation of the whole L2 per workgroup: measured 25.3 us against 21.9 us.
    __hip_atomic_store(out, o0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(out + 1, o1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // the compiler may move nothing across the wait: the stores stay above it, the ticket below
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_s_waitcnt(0);
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    // the ticket is drawn: this thread's second atomic on the word after the one that raised it to the launch's
    // epoch, two atomics of one thread on one address, applied in program order
    uint64_t ticket = __hip_atomic_fetch_add(my_word, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    bool last = ticket == base + my_arrivals - 1u;
    if (grouped && last) {
      // last of its group: the group's word goes back to zero (as the row's word below), and the group arrives at
      // the row's word, which its first arrival raises
      __hip_atomic_store(my_word, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_fetch_max(counters + b, base, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      ticket = __hip_atomic_fetch_add(counters + b, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const int n_groups = nblk < kRelL1Groups ? nblk : kRelL1Groups;
      last = ticket == base + static_cast<uint64_t>(n_groups) - 1u;
    }
    last_of_row = last;
    __atomic_signal_fence(__ATOMIC_SEQ_CST);  // the reader's loads below stay below the ticket
  }
  __syncthreads();
  if (!last_of_row) return;  // uniform over the workgroup

  // ---- last workgroup of row b: every partial of the row has landed (see above) ----
  const float2* pr = reinterpret_cast<const float2*>(partials) + static_cast<int64_t>(b) * nblk;
  // fixed assignment partial i -> thread i % NT, all loads of a thread independent
  double dd = 0.0, dp = 0.0;
  for (int i = threadIdx.x; i < nblk; i += NT) {
    dd += __hip_atomic_load(&pr[i].x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    dp += __hip_atomic_load(&pr[i].y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    dd += __shfl_xor(dd, off, 64);
    dp += __shfl_xor(dp, off, 64);
  }
  __shared__ double red2[2][NWAVE];
  if ((threadIdx.x & 63) == 0) { red2[0][wave] = dd; red2[1][wave] = dp; }
  __syncthreads();
  if (threadIdx.x == 0) {
    double t0 = 0.0, t1 = 0.0;
#pragma unroll
    for (int w = 0; w < NWAVE; ++w) { t0 += red2[0][w]; t1 += red2[1][w]; }
    sums[2 * b] = t0;
    sums[2 * b + 1] = t1;
    // back to zero: a launch recorded in a HIP graph is replayed with the same epoch, and finds its word as
    // the first launch did
    __hip_atomic_store(counters + b, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// Puts n ticket words to zero (a kernel, not a memset: safe to record into a HIP graph).
__global__ __launch_bounds__(256) void rel_l1_clear_kernel(uint64_t* counters, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) counters[i] = 0ull;
}

template <typename T>
static int launch_rel_l1(const void* cur, const void* prev, double* sums, uint64_t* counters, uint64_t* groups, float* partials, int B,
                         int64_t n, int64_t cur_stride, int64_t prev_stride, bool ref_round,
                         hipStream_t stream) {
  constexpr int EPV = Vec16<T>::N;
  const bool vec_ok = aligned16(cur) && aligned16(prev) && cur_stride % EPV == 0 &&
                      prev_stride % EPV == 0;
  const int64_t n_vec = vec_ok ? n / EPV : 0;
  const int nblk = rel_l1_blocks_per_row(B, n);
  const uint64_t epoch = next_ticket_epoch();
  const dim3 grid(nblk, B);
  if (ref_round) {
    hipLaunchKernelGGL((rel_l1_kernel<T, true>), grid, dim3(kRelL1Threads), 0, stream, static_cast<const T*>(cur),
                       static_cast<const T*>(prev), partials, counters, groups, epoch, sums, n, n_vec, cur_stride, prev_stride);
  } else {
    hipLaunchKernelGGL((rel_l1_kernel<T, false>), grid, dim3(kRelL1Threads), 0, stream, static_cast<const T*>(cur),
                       static_cast<const T*>(prev), partials, counters, groups, epoch, sums, n, n_vec, cur_stride, prev_stride);
  }
  return check_launch("odit_rel_l1");
}

static size_t rel_l1_partial_bytes(int B, int64_t n) {
  return static_cast<size_t>(B) * rel_l1_blocks_per_row(B, n) * 2 * sizeof(float);
}

}  // namespace odit

extern "C" size_t odit_rel_l1_workspace_bytes(int B, int64_t n) {
  if (B <= 0 || n < 0) return 0;
  return odit::kRelL1CounterBytes + odit::rel_l1_partial_bytes(B, n);
}

extern "C" int odit_rel_l1(const void* cur, const void* prev, double* sums, void* workspace,
                           size_t workspace_bytes, int B, int64_t n, int64_t cur_stride,
                           int64_t prev_stride, int dtype, unsigned flags, void* stream) {
  using namespace odit;
  ODIT_CHECK_ARG(cur && prev && sums && workspace, "odit_rel_l1: null pointer argument");
  ODIT_CHECK_ARG(B > 0 && B <= kRelL1MaxRows && n >= 0, "odit_rel_l1: bad shape B=%d n=%lld", B,
                 static_cast<long long>(n));
  ODIT_CHECK_ARG(aligned16(workspace), "odit_rel_l1: workspace must be 16-byte aligned");
  if (workspace_bytes < odit_rel_l1_workspace_bytes(B, n)) {
    set_error("odit_rel_l1: workspace has %zu bytes, needs %zu", workspace_bytes,
              odit_rel_l1_workspace_bytes(B, n));
    return ODIT_EWORKSPACE;
  }
  const bool rr = (flags & ODIT_FLAG_REF_ROUNDING) && dtype != ODIT_F32;
  uint64_t* counters = static_cast<uint64_t*>(workspace);
  uint64_t* groups = reinterpret_cast<uint64_t*>(static_cast<char*>(workspace) + kRelL1RowWordBytes);
  float* partials = reinterpret_cast<float*>(static_cast<char*>(workspace) + kRelL1CounterBytes);
  ODIT_DISPATCH_DTYPE(dtype, T,
                      return launch_rel_l1<T>(cur, prev, sums, counters, groups, partials, B, n, cur_stride, prev_stride, rr,
                                              static_cast<hipStream_t>(stream)));
  return ODIT_OK;
}

// ---------------------------------------------------------------------------------------------
// The same reduction for callers that cannot allocate: its scratch is a fixed array in device memory
// (one copy per GPU the library runs on, held until the process ends).
namespace odit {

// 512 bytes of ticket words + one float pair per workgroup: a launch over at most kRelL1StaticRows rows has at most
// kRelL1TotalBlocks workgroups (rel_l1_blocks_per_row), so 2560 bytes hold any call this entry point accepts
constexpr size_t kRelL1StaticCounterBytes = kRelL1StaticRows * sizeof(uint64_t);
constexpr size_t kRelL1StaticBytes = kRelL1StaticCounterBytes + static_cast<size_t>(kRelL1TotalBlocks) * 2 * sizeof(float);
static_assert(kRelL1StaticCounterBytes % 256 == 0, "the partials start on a 256-byte boundary");
static_assert(kRelL1StaticRows <= kRelL1TotalBlocks, "one workgroup per row at least");

static __device__ __align__(256) unsigned char scratch[kRelL1StaticBytes];

// The array's name is only a host-side handle; its device address differs per GPU and is looked up once
// per device, with that device current, and kept.
static void* static_scratch_ptr(int* status) {
  constexpr int kMaxDevices = 64;
  static void* ptrs[kMaxDevices] = {nullptr};
  static std::mutex mu;
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    set_error("odit_rel_l1_static: cannot tell the current device (%s)", hipGetErrorString(e));
    *status = ODIT_ELAUNCH;
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(mu);
  if (ptrs[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
      set_error("odit_rel_l1_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
      *status = ODIT_ELAUNCH;
      return nullptr;
    }
    ptrs[dev] = p;
  }
  *status = ODIT_OK;
  return ptrs[dev];
}

}  // namespace odit

extern "C" void* odit_rel_l1_static_scratch(size_t* bytes) {
  int rc = ODIT_OK;
  void* ptr = odit::static_scratch_ptr(&rc);
  if (bytes != nullptr) *bytes = ptr != nullptr ? odit::kRelL1StaticBytes : 0;
  return ptr;
}

extern "C" int odit_rel_l1_static(const void* cur, const void* prev, double* sums, int B, int64_t n,
                                  int64_t cur_stride, int64_t prev_stride, int dtype, unsigned flags,
                                  void* stream) {
  using namespace odit;
  ODIT_CHECK_ARG(cur && prev && sums, "odit_rel_l1_static: null pointer argument");
  ODIT_CHECK_ARG(B > 0 && n >= 0, "odit_rel_l1_static: bad shape B=%d n=%lld", B, static_cast<long long>(n));
  if (B > kRelL1StaticRows) {
    set_error("odit_rel_l1_static: B=%d rows exceed the %d rows the built-in scratch holds; use odit_rel_l1 with "
              "a workspace", B, kRelL1StaticRows);
    return ODIT_EWORKSPACE;
  }
  if (kRelL1StaticCounterBytes + rel_l1_partial_bytes(B, n) > kRelL1StaticBytes) {  // cannot happen while the row limit holds
    set_error("odit_rel_l1_static: %zu bytes of scratch needed, %zu built in",
              kRelL1StaticCounterBytes + rel_l1_partial_bytes(B, n), kRelL1StaticBytes);
    return ODIT_EWORKSPACE;
  }
  int rc = ODIT_OK;
  void* ptr = static_scratch_ptr(&rc);
  if (ptr == nullptr) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // The array keeps whatever the last call left (normally ticket words back at zero; not if that call's kernel
  // never finished): clear this call's ticket words first. A fill kernel, not a memset, so the pair may be captured in a graph.
  hipLaunchKernelGGL(rel_l1_clear_kernel, dim3(1), dim3(256), 0, st, static_cast<uint64_t*>(ptr), kRelL1StaticRows);
  rc = check_launch("odit_rel_l1_static (clear)");
  if (rc != ODIT_OK) return rc;
  const bool rr = (flags & ODIT_FLAG_REF_ROUNDING) && dtype != ODIT_F32;
  uint64_t* counters = static_cast<uint64_t*>(ptr);
  float* partials = reinterpret_cast<float*>(static_cast<char*>(ptr) + kRelL1StaticCounterBytes);
  ODIT_DISPATCH_DTYPE(dtype, T,
                      return launch_rel_l1<T>(cur, prev, sums, counters, nullptr, partials, B, n, cur_stride, prev_stride, rr, st));
  return ODIT_OK;
}
