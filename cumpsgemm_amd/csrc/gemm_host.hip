// Host side of the GEMM path: handle life cycle, tile selection, launches and
// the C ABI.  Takes the place of reference src/handle.cu:7-52 and
// src/cumpsgemm.cu:19-605.
#include "gemm_table.hpp"
#include "handle.hpp"
#include "pack_split.hpp"
#include "utils.hpp"
#include <cumpsgemm/cumpsgemm.hpp>
#include <cumpsgemm/cumpsgemm_ext.h>
#include <mutex>
#include <new>
#include <stdexcept>
#include <type_traits>

namespace cumpsgemm_amd {

namespace {
Tuning read_tuning_env() {
  Tuning t;
  auto as_int = [](const char *name, int unset) {
    const char *v = std::getenv(name);
    return v != nullptr ? std::atoi(v) : unset;
  };
  if (const char *v = std::getenv("CUMPSGEMM_PACKED")) t.packed = v[0] == '0' ? 0 : (v[0] == '1' ? 1 : -1);
  if (const char *v = std::getenv("CUMPSGEMM_PACKED_WALK")) t.packed_walk = v[0] == '1' ? 1 : 0;
  const int rg = as_int("CUMPSGEMM_RASTER_GROUP", 0);
  t.raster_group = (rg >= 1 && rg <= 64) ? rg : 0;
  t.fetch_from_one_patch = std::getenv("CUMPSGEMM_EXP_FETCH_FROM_ONE_PATCH") != nullptr;
  t.force_cls = as_int("CUMPSGEMM_FORCE_TILE_CLASS", -1);
  if (t.force_cls < 0 || t.force_cls >= kNumTileClasses) t.force_cls = -1;
  t.force_split = as_int("CUMPSGEMM_FORCE_KSPLIT", 0);
  t.no_persistent = std::getenv("CUMPSGEMM_NO_PERSISTENT") != nullptr;
  t.no_column_split = std::getenv("CUMPSGEMM_NO_COLUMN_SPLIT") != nullptr;
  t.cut_percent = as_int("CUMPSGEMM_CUT_PERCENT", t.cut_percent);
  t.no_kslices = std::getenv("CUMPSGEMM_NO_KSLICE_GROUPS") != nullptr;
  t.no_edge16_twin = std::getenv("CUMPSGEMM_NO_EDGE16_TWIN") != nullptr;
  t.no_fused_scaling = std::getenv("CUMPSGEMM_NO_FUSED_SCALING") != nullptr;
  if (const char *v = std::getenv("CUMPSGEMM_PERSISTENT_MAX_STEPS")) t.persistent_max_steps = (unsigned)std::atoi(v);
  if (const char *v = std::getenv("CUMPSGEMM_MAX_WORKSPACE_BYTES")) t.max_workspace_bytes = std::strtoull(v, nullptr, 10);
  return t;
}
// The current snapshot of the tuning variables.  A reload publishes a new,
// immutable object and leaves the old one in place (never freed: a few dozen
// bytes per reload, and reloads are a test facility), so a thread that took a
// reference before the reload keeps reading a consistent set of values.
std::atomic<unsigned long long *> g_walk_stamps{nullptr}; // (diagnostic builds only)
std::atomic<const Tuning *> g_tuning{nullptr};
std::mutex g_tuning_mutex;
} // namespace

// ---- home of the pre-split planes for the entry point that allocates nothing
// One array per GPU, inside the library's code object, held until the process
// ends.  In host code `scratch` is only a stand-in for the symbol: the device
// address is asked for once per device (scratch_address) and that pointer is
// what kernels and the planner get.
constexpr unsigned long long kStaticScratchBytes = 64ull << 20;
} // namespace cumpsgemm_amd
static __device__ __align__(256) unsigned char scratch[cumpsgemm_amd::kStaticScratchBytes];
namespace cumpsgemm_amd {
namespace {
constexpr int kMaxDevices = 64;
void *g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;
// Device address of `scratch` on device `dev`, which must be the current
// device; nullptr (logged) if the runtime cannot resolve it.
void *scratch_address(int dev) {
  if (dev < 0 || dev >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void *ptr = nullptr;
    const hipError_t err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess || ptr == nullptr) {
      (void)hipGetLastError();
      log_error(std::string("hipGetSymbolAddress(scratch) failed: ") + hipGetErrorString(err));
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
    // the kernels that entry point launches are loaded now, so that its first
    // call does not make the runtime allocate memory for their code either
    prepare_pack_split_real();
    prepare_packed_fp16tcec_s();
    prepare_packed_bf16x3_s();
  }
  return g_scratch_ptr[dev];
}
} // namespace

const Tuning &tuning() {
  const Tuning *t = g_tuning.load(std::memory_order_acquire);
  if (t == nullptr) {
    std::lock_guard<std::mutex> lock(g_tuning_mutex);
    t = g_tuning.load(std::memory_order_acquire);
    if (t == nullptr) {
      t = new Tuning(read_tuning_env());
      g_tuning.store(t, std::memory_order_release);
    }
  }
  return *t;
}

void check_hip(hipError_t err, const char *what) {
  if (err != hipSuccess) {
    const std::string msg = std::string(what) + ": " + hipGetErrorString(err);
    log_error(msg);
    throw std::runtime_error(msg);
  }
}

ProfileScope::ProfileScope(cuMpSGEMM_handle *handle, const char *label)
    : h(handle), name(label) {
  if (h->profiler.enabled) {
    (void)hipStreamSynchronize(h->stream);
    h->profiler.t0 = std::chrono::steady_clock::now();
  }
}
ProfileScope::~ProfileScope() {
  if (h->profiler.enabled) {
    (void)hipStreamSynchronize(h->stream);
    const auto t1 = std::chrono::steady_clock::now();
    auto &e = h->profiler.entries[name];
    e.sum += std::chrono::duration<double>(t1 - h->profiler.t0).count();
    e.n++;
  }
}

const KernelEntry *lookup_kernel(Prec p, bool cplx, bool a_kc, bool b_kc, int cls) {
  const int layout = (a_kc ? 1 : 0) + (b_kc ? 2 : 0);
  switch (p) {
  case Prec::FP16TCEC:
    return cplx ? &g_tab_fp16tcec_c[layout][cls] : &g_tab_fp16tcec_s[layout][cls];
  case Prec::FP16TC:
    return cplx ? &g_tab_fp16tc_c[layout][cls] : &g_tab_fp16tc_s[layout][cls];
  case Prec::BF16X3:
    return cplx ? &g_tab_bf16x3_c[layout][cls] : &g_tab_bf16x3_s[layout][cls];
  case Prec::BF16X2:
    return cplx ? &g_tab_bf16x2_c[layout][cls] : &g_tab_bf16x2_s[layout][cls];
  }
  return nullptr;
}

namespace {
__global__ void init_rings_kernel(StatsSlot *slots, int *flags, unsigned *ticket) {
  // presets of the reference: stats slot 0 -> TF32TCEC, slot 1 -> FP16TCEC
  // (src/exp_stats.cu:496-499); flag slot 0 -> TF32TCEC, slot 1 -> FP16TCEC with
  // both scale bits (src/dynamic_launch.cu:6-9)
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    slots[0].mode = CUMPSGEMM_TF32TCEC;
    slots[1].mode = CUMPSGEMM_FP16TCEC;
    flags[0] = CUMPSGEMM_TF32TCEC;
    flags[1] = (3 << 5) | CUMPSGEMM_FP16TCEC;
    ticket[0] = 0;
    ticket[1] = 0;
    ticket[2] = 0;
  }
}

bool mode_to_prec(cuMpSGEMM_compute_mode_t mode, Prec &p) {
  switch (mode) {
  case CUMPSGEMM_FP16TCEC:
  case CUMPSGEMM_FP16TCEC_SCALING: // scaling is orchestrated outside the kernel
    p = Prec::FP16TCEC;
    return true;
  case CUMPSGEMM_FP16TC:
    p = Prec::FP16TC;
    return true;
  case CUMPSGEMM_TF32TCEC:
    p = Prec::BF16X3;
    return true;
  case CUMPSGEMM_TF32TC:
    p = Prec::BF16X2;
    return true;
  default:
    return false;
  }
}

struct Plan {
  const KernelEntry *entry;
  int cls;
  unsigned tiles_m, tiles_n, ksplit, k_chunk;
  double cost; // of the cost model below; comparable between shapes
};

// workgroups of this kernel that one CU holds at a time
unsigned resident_groups(const KernelEntry *e) {
  const unsigned by_lds = (160u * 1024u) / (unsigned)e->lds_bytes;
  const unsigned by_regs = (unsigned)(e->occ * 4 * 64) / (unsigned)e->threads;
  const unsigned r = by_lds < by_regs ? by_lds : by_regs;
  return r < 1 ? 1 : r;
}

// Shape -> tile class and split-K factor.  The reference fills "two waves of
// SMs" with its first candidate or falls back to the second, and splits K for
// small outputs (src/cumpsgemm.cu:242-253, x32 for batches :453-454).  Here
// every (class, split) pair gets a cost from a small model fitted to
// measurements on MI355X, and the cheapest wins:
//   cost = rounds * (K-steps per chunk + F) * tile area * resident groups / efficiency
//          [+ a fixed charge when K is split]
// rounds     = how many times the chip's CU slots must be refilled (a problem
//              smaller than one round is charged for the workgroups a CU
//              really holds),
// + F        = a tile's fixed cost (pipeline fill, write-out) in K-steps: 5 for
//              the 256x128 tiles, 3 for 128x128, 4 for the others (FP16TC, a
//              third of the MFMAs per step: 4 throughout; complex: 3 for 128x64,
//              4 for the others; the tables whose large tile uses 16x16x32
//              MFMAs in the K loop: 6 and 4),
// efficiency = sustained MFMA rate relative to the 64x64 wave tile, which has
//              the fewest LDS fragment reads per MFMA (64x32: 0.83, 32x32: 0.55,
//              less when a CU holds under two waves per SIMD; the in-loop large
//              tiles with 16x16x32 MFMAs: 1.1; the complex 64x64 and 64x32
//              tiles, which are not persistent: x 0.8),
// (F and the efficiencies were fitted on 34 shapes x 3 layouts x {FP16TCEC, bf16x3}, single
// and strided-batch, each timed with every class forced: with F = 4 throughout the
// model kept the large tile for batches of small matrices and for K <= 256,
// where 128x128 measures 5 - 30 % faster -- 384^3 x 128 201 -> 226, 4096^2 x 128
// 162 -> 175, 768^3 x 32 NT 199 -> 240, bf16x3 512^2 x 128 x 128 116 -> 131 TFLOP/s;
// the sum of the relative losses against the best class fell from 2.6 to 0.73
// (FP16TCEC) and from 3.8 to 1.2 (bf16x3); complex FP16TCEC 1.3 -> 0.53 -- 320^3 x 256
// 208 -> 250, 1024^2 x 4096 NT 221 -> 283 TFLOP/s --, complex bf16x3 0.73 -> 0.06;
// FP16TC fits best with what it had.  The 256x128 kernels of bf16x2 and the 128x256
// one of FP16TCEC were then rebuilt on 16x16x32 MFMAs -- bf16x2 512^3 x 64 213 -> 305,
// 4096^2 x 512 221 -> 310, FP16TCEC NT 1024^3 x 8 256 -> 324 TFLOP/s -- and their
// tables fitted again: 6 / 4 K-steps, 1.1.)
// split charge = the extra launch that prepares C (about four K-steps of the
//              largest tile; real: one) plus the atomic write-out, which grows
//              with the number of chunks adding into the same C.
// K-chunks are multiples of the 32-wide step and at least four steps long.
Plan make_plan(const cuMpSGEMM_handle *h, Prec p, bool cplx, bool a_kc, bool b_kc,
               uint64_t m, uint64_t n, uint64_t k, uint64_t batch, int force_cls, int force_split) {
  Plan plan{};
  int cls = 0;
  unsigned ksplit = 1;
  double best = -1.0;
  const uint64_t nk = (k + 31) / 32;
  const uint64_t max_split = std::max<uint64_t>(1, std::min<uint64_t>(k / 128, 64));
  uint64_t forced_split = 0; // largest power of two <= min(force_split, max_split)
  if (force_split > 0) {
    forced_split = 1;
    while (forced_split * 2 <= (uint64_t)force_split && forced_split * 2 <= max_split) forced_split *= 2;
  }
  for (int c = 0; c < kNumTileClasses; c++) {
    if (force_cls >= 0 && c != force_cls) continue;
    const KernelEntry *e = lookup_kernel(p, cplx, a_kc, b_kc, c);
    const uint64_t tiles = ((m + e->bm - 1) / e->bm) * ((n + e->bn - 1) / e->bn) * batch;
    const unsigned res = resident_groups(e);
    const uint64_t slots = (uint64_t)h->num_cus * res;
    const int wave_area = e->wm * e->wn;
    // efficiency with `groups` workgroups on a CU: the 32x32 wave tiles need
    // two waves per SIMD to hide their own latencies (0.52 us per K-step for a
    // lone 4-wave 64x64 workgroup, 0.65 us for two of them side by side)
    // (tables whose large tile multiplies with 16x16x32 MFMAs in the K loop: real bf16x2, and
    // real FP16TCEC when both operands are M/N-contiguous)
    const bool edge16_table = !cplx && (p == Prec::BF16X2 || (p == Prec::FP16TCEC && !a_kc && !b_kc));
    const int tile_elems = e->bm * e->bn;
    const bool cplx_large = cplx && tile_elems >= 128 * 64;
    const double fixed_steps = cplx ? (cplx_large ? 3.0 : 4.0)
                               : (p == Prec::FP16TC ? 4.0
                                  : (tile_elems >= 256 * 128 ? (edge16_table ? 6.0 : 5.0)
                                                             : (tile_elems >= 128 * 128 ? (edge16_table ? 4.0 : 3.0) : 4.0)));
    const double small_cplx = (cplx && !cplx_large) ? 0.8 : 1.0;
    auto eff_of = [&](double groups, bool whole_rounds = false) {
      if (wave_area >= 4096) return edge16_table ? 1.1 : 1.0;
      if (wave_area >= 2048) return 0.83;
      const double waves_per_simd = (double)e->threads * groups / 256.0;
      if (cplx) return small_cplx * (waves_per_simd >= 2.0 ? 0.55 : (waves_per_simd >= 1.0 ? 0.375 : 0.19));
      // (real 64x64 tiles, fitted on 22 shapes from 256^3 to 1536^3 and 896^2 x 2048 x 4 layouts x
      // {FP16TCEC, bf16x3} x {class 1, 2} x {K split 1, 2, 4, 8}: a lone workgroup on a CU runs as
      // two wave groups when an operand is K-contiguous)
      // (whole rounds of a chip full of small workgroups: 0.55 -- with 0.65 there, batches of 320^3
      // matrices took 64x64 tiles at half the rate of 128x128)
      return waves_per_simd >= 2.0 ? (whole_rounds ? 0.55 : 0.65)
                                   : (waves_per_simd >= 1.0 ? ((a_kc || b_kc) ? 0.45 : 0.375) : 0.19);
    };
    // (a tile's operand traffic per flop grows with 1/bm + 1/bn: charged lightly,
    // which also settles ties in favour of the larger tile)
    const double area = (double)e->bm * e->bn * (1.0 + 2.0 / e->bm + 2.0 / e->bn);
    const double unit = area * res / eff_of((double)res, true);
    const double atomics = (double)m * (double)n * (double)batch * (cplx ? 2.0 : 1.0);
    for (uint64_t sp = 1; sp <= max_split; sp *= 2) {
      if (forced_split != 0 && sp != forced_split) continue;
      // a problem that does not fill the CU slots once keeps fewer workgroups on
      // a CU than could live there; otherwise whole rounds are charged
      const uint64_t groups = tiles * sp;
      const double steps = (double)((nk + sp - 1) / sp) + fixed_steps;
      double cost;
      if (groups <= slots) { // (one round at most: the workgroups of a CU start together)
        const double per_cu = (double)((groups + h->num_cus - 1) / h->num_cus);
        cost = steps * per_cu * area / eff_of(per_cu);
      } else {
        cost = steps * (double)((groups + slots - 1) / slots) * unit;
      }
      // (real: fitted with the efficiencies above; the larger charge kept 896^2 x 2048 unsplit at 32 - 59 us
      // where two K-chunks take 25 - 28, and 512^3 ... 1024^3 with two M/N-contiguous operands 10 - 50 % slow)
      if (sp > 1) cost += cplx ? 4.0 * 256.0 * 128.0 + 0.1 * atomics * (double)sp
                               : 256.0 * 128.0 + 0.05 * atomics * (double)sp;
      if (best < 0.0 || cost < best) {
        best = cost;
        cls = c;
        ksplit = (unsigned)sp;
      }
      if (forced_split == 0 && tiles * sp >= slots) break; // more chunks would only add rounds
    }
  }
  const KernelEntry *e = lookup_kernel(p, cplx, a_kc, b_kc, cls);
  plan.entry = e;
  plan.cls = cls;
  plan.tiles_m = (unsigned)((m + e->bm - 1) / e->bm);
  plan.tiles_n = (unsigned)((n + e->bn - 1) / e->bn);
  unsigned k_chunk = (unsigned)((k + ksplit - 1) / ksplit);
  k_chunk = (k_chunk + 31) / 32 * 32;
  ksplit = (unsigned)((k + k_chunk - 1) / k_chunk);
  plan.ksplit = ksplit;
  plan.k_chunk = k_chunk;
  plan.cost = best;
  return plan;
}

// The persistent kernels load without guards: the matrix must be at least one
// tile wide and high (edge tiles are computed from an origin moved inwards),
// every K-chunk a multiple of the 32-wide step and at least four steps long,
// and every per-thread offset must fit 31 bits.
// (K-steps per tile up to which tiles are walked: Tuning::persistent_max_steps, 32)
unsigned persistent_max_steps() { return tuning().persistent_max_steps; }

template <class T>
bool persistent_ok(const KernelEntry *e, bool a_kc, bool b_kc, uint64_t m, uint64_t n, uint64_t k,
                   const Plan &plan, uint64_t lda, uint64_t ldb, uint64_t batch, bool any_length) {
  constexpr uint64_t ES = sizeof(T) / sizeof(float);
  if (m < (uint64_t)e->bm || n < (uint64_t)e->bn || k % 32 != 0) return false;
  const uint64_t last_chunk = k - (uint64_t)(plan.ksplit - 1) * plan.k_chunk;
  if (plan.k_chunk % 32 != 0 || plan.k_chunk < 128 || last_chunk < 128) return false;
  // Walking tiles pays while a tile is short: the next tile's first steps load
  // during the write-out.  Long tiles gain nothing from that and run 1 - 4 %
  // faster as independent workgroups, which drift apart in time instead of
  // asking memory for the same K range in lockstep.  (The kernels with fused
  // scaling are the exception: their one-tile form measures 7 % slower for the
  // NN layout, so they walk tiles of any length.)
  if (!any_length && plan.k_chunk / 32 > persistent_max_steps()) return false;
  auto fits = [&](bool kc, uint64_t rows, uint64_t ld) {
    const uint64_t span = kc ? rows * ld + 32 : 32 * ld + rows;
    return span * ES * 4 < 0x7fffffffull;
  };
  if (!fits(a_kc, (uint64_t)e->bm, lda) || !fits(b_kc, (uint64_t)e->bn, ldb)) return false;
  if ((uint64_t)plan.tiles_m * plan.tiles_n * batch > 0x7fffffffull) return false;
  return true;
}

template <class T> struct scalar_parts;
template <> struct scalar_parts<float> {
  static void get(const float *s, float &re, float &im) { re = *s; im = 0.0f; }
};
template <> struct scalar_parts<hipComplex> {
  static void get(const hipComplex *s, float &re, float &im) { re = s->x; im = s->y; }
};

// ---------------------------------------------------------------------------
// Pre-split path (FP16TCEC real and complex; bf16x3, FP16TC and bf16x2 real): split A and B once,
// up front, into fp16 / bf16 planes held in the handle's workspace, and run the
// kernel that only copies them into LDS.  Same split and same products as the
// in-loop kernels; the order of summation differs (16x16x32 MFMAs add 32
// K-values at a time, the in-loop kernels' 32x32x16 MFMAs 16), so results agree
// to a few FP32 roundings, not bit for bit.  The pre-pass is one
// read + write of A and B at 5 - 6 TB/s; what it buys is a K loop without split
// arithmetic, which runs at a higher clock under the power limit.  It pays for
// large problems (rules below, per mode and layout); the in-loop kernels serve
// the rest and need no workspace.  CUMPSGEMM_PACKED=1 / 0 forces / forbids it.
enum class PreSplit {
  NOT_TAKEN,   // the caller launches the in-loop kernels
  DONE,        // C is (being) computed; nothing left to launch
  FP16_SERVED, // AUTO: the FP16TCEC candidate is launched, bf16x3 is left to the caller
  FAILED       // a launch or the stream failed (logged)
};

struct PreSplitChoice {
  bool take = false;
  bool bf16 = false;      // explicit TF32TCEC: three bf16 planes
  bool tc_only = false;   // FP16TC / TF32TC (no correction terms): one fp16 plane / two bf16 planes
  bool auto_ok = false;   // AUTO: the gated FP16TCEC candidate goes this way
  bool auto_bf16 = false; // AUTO: and so does the gated bf16x3 candidate
  // not taken only because the last round of CU slots would be mostly empty:
  // worth taking for the part of C that fills whole rounds
  bool cut = false;
  int bm = 0, bn = 0;     // tile of the kernel that reads the planes
  unsigned planes = 0;    // planes per K-step of one operand
};

template <bool CPLX>
PreSplitChoice choose_pre_split(const cuMpSGEMM_handle *h, bool a_kc, bool b_kc, uint64_t m, uint64_t n,
                                uint64_t k, uint64_t batch, cuMpSGEMM_compute_mode_t mode,
                                int force_cls, int force_split, int depth) {
  PreSplitChoice ch;
  ch.tc_only = mode == CUMPSGEMM_FP16TC || mode == CUMPSGEMM_TF32TC;
  if (CPLX && mode != CUMPSGEMM_FP16TCEC && mode != CUMPSGEMM_TF32TCEC && !ch.tc_only) return ch; // (AUTO: real only)
  // CUMPSGEMM_PACKED: "0" never, "1" whenever possible; the entry point that
  // allocates nothing always goes this way (its planes have a home already)
  const bool forced = h->ws_override != nullptr;
  // (depth 2: the whole rounds of a problem that was cut for this path)
  const bool never = tuning().packed == 0 && !forced, always = tuning().packed == 1 || forced || depth == 2;
  // bf16x3 (explicit TF32TCEC mode): its in-loop three-way split costs 5.4
  // vector instructions per MFMA, so the pre-pass pays for every layout
  ch.bf16 = (mode == CUMPSGEMM_TF32TCEC);
  ch.bm = CPLX ? kPackedCplxBM : (ch.bf16 ? kPackedBf16BM : kPackedBM);
  ch.bn = CPLX ? kPackedCplxBN : (ch.bf16 ? kPackedBf16BN : kPackedBN);
  ch.planes = (CPLX ? 2u : 1u) * (ch.bf16 ? 3u : (mode == CUMPSGEMM_FP16TC ? 1u : 2u));
  // (complex bf16x3: the 128x64 complex tile, like the other complex modes)
  // (the pre-pass launches workgroups of 64 rows x 32 .. 256 K-values on a 2-D grid)
  const bool shape_ok = batch == 1 && k >= 128 &&
                        (forced || (uint64_t)m * n >= (uint64_t)h->num_cus * ch.bm * ch.bn) && k / 32 < 65535;
  const double mn_ratio = (double)m * (double)n / ((double)m + (double)n);
  // (in-loop -> pre-split, TFLOP/s: 4096^2 x 256 198 -> 211, 4096^2 x 384 224 -> 260, 5120^2 x 256 176 -> 209,
  // 3072^2 x 512 177 -> 191, 3072^2 x 1024 201 -> 237, 8192 x 4096 x 256 211 -> 245, 4096 x 8192 x 384 232 -> 316;
  // 3072^2 x 2048 level)
  const bool pays_nt_shape = !a_kc && !b_kc && ((k >= 384 && mn_ratio >= 1500.0) || (k >= 256 && mn_ratio >= 2000.0));
  // Every other layout: the pre-split kernel, freed of the split arithmetic,
  // outruns the in-loop one by more than the pre-pass costs once the problem
  // is large (8192^3: 381 vs 361 - 372 TFLOP/s; 8192^2 x 1024: 351 vs 318 -
  // 343) -- provided the last round of CU slots is at least half full or one
  // of many: the path has no column split for a mostly empty last round.
  const uint64_t ptiles = ((m + ch.bm - 1) / ch.bm) * ((n + ch.bn - 1) / ch.bn);
  const uint64_t last_round = ptiles % h->num_cus;
  const bool rounds_ok = last_round == 0 || 2 * last_round >= h->num_cus || ptiles >= 6ull * h->num_cus;
  // (complex: four times the MFMA work per element split, so the pre-pass weighs less)
  // (5120^3, 800 tiles = 3.1 rounds: 329 TFLOP/s this way, 356 in-loop, whose planner cuts C in two)
  // With fused scaling the in-loop split costs one more instruction per pair
  // and those kernels run 8 - 25 % below the plain ones, so the pre-pass (which
  // scales as it splits) pays for every layout.
  const bool pays_scaled = h->fused_scaling && k >= 256 && mn_ratio >= 1800.0;
  // AUTO: the FP16TCEC candidate may take the path as well, gated by the
  // launch flag like every AUTO kernel (pre-pass included).  Both candidates
  // write C directly, which needs the bf16x3 plan to be free of split-K.
  if (!CPLX && mode == CUMPSGEMM_AUTO && pays_scaled && depth == 0) {
    ch.auto_ok = make_plan(h, Prec::BF16X3, CPLX, a_kc, b_kc, m, n, k, batch, force_cls, force_split).ksplit == 1;
  }
  // (measured against the in-loop 256x128 class, NN / TN, TFLOP/s: 8192^2 x 256 167 / 172 -> 189 / 187,
  // 6144^2 x 256 152 / 157 -> 173 / 178, 4096^2 x 512 182 / 189 -> 190 / 191, 4096^3 208 / 213 -> 231 / 228,
  // 3072^2 x 1024 157 / 162 -> 171 / 171, 2048^2 x 2048 188 / 178 -> 200 / 198; 4096^2 x 384, 3072^2 x 512 and
  // 2048^2 x 1024 are level, shorter K loses)
  const bool pays_bf16 = (k >= 256 && mn_ratio >= 3000.0) || (k >= 512 && mn_ratio >= 2000.0) ||
                         (k >= 1024 && mn_ratio >= 1500.0) || (k >= 2048 && mn_ratio >= 1000.0);
  // The rules that depend on how well the rounds of CU slots are filled (ro:
  // rounds_ok, or taken for granted to see whether a cut of C would pay).
  auto worth_if = [&](const bool ro) {
    const bool pays_nt = pays_nt_shape && ro;
    // Shorter K: per tile the in-loop kernels lose more to the split than the pre-pass
    // costs once C is large (in-loop -> pre-split, TFLOP/s, NN / TN: 8192^2 x 256 261 / 270 -> 277 / 278,
    // 8192^2 x 384 287 / 297 -> 314 / 313, 6144^2 x 384 254 / 266 -> 280 / 282, 6144^2 x 512 274 / 285 -> 306 / 307,
    // 4096^2 x 1024 326 / 333 -> 343 / 343, 4096^2 x 2048 350 / 357 -> 384 / 384; 6144^2 x 256 and 4096^2 x 512
    // are level and stay in-loop, 4096^2 x 256 would lose 8 - 11 %).
    // (re-measured with the cheaper write-out of the pre-split kernels, NN / TN, packed over in-loop: 4096^2 x 384
    // 1.00 / 0.99, 4096 x 8192 x 384 1.12 / 1.14, 6144^2 x 384 1.06 / 1.04, 4096^2 x 512 1.01 / 1.01, 4096^2 x 768
    // 1.08 / 1.07, 6144^2 x 256 1.06 / 1.01, 8192 x 4096 x 256 0.96 / 0.95, 5120^2 x 256 0.91 / 0.90)
    const bool pays_short = !CPLX && ro &&
                            ((k >= 256 && mn_ratio >= 4000.0) || (k >= 384 && mn_ratio >= 2500.0) ||
                             (k >= 768 && mn_ratio >= 2000.0));
    // (complex, in-loop -> pre-split, NN / TN: 4096^3 367 / 378 -> 432 / 435 TFLOP/s, 2048^3 355 / 364 -> 401 / 400,
    // 2048^2 x 1024 349 / 347 -> 372 / 374, 3072^2 x 384 309 / 314 -> 329 / 325, 4096^2 x 256 313 / 320 -> 342 / 349,
    // 8192^2 x 256 323 / 321 -> 368 / 373; 2048^2 x 512 level, 2048^2 x 384 would lose 5 %, 3072^2 x 256 level)
    // (re-measured with the cheaper write-out, packed over in-loop, NN / TN / NT: 2048^2 x 512 1.03 / 1.02 / 1.10,
    // 2048^2 x 768 1.06 / 1.04 / 1.06, 2560^2 x 384 1.03 / 1.05 / 1.09, 3072^2 x 256 1.03 / 1.03 / 1.05; 2048^2 x 384
    // 0.98 / 0.95 / 1.03, 2560^2 x 256 0.96 / 0.97 / 1.00, 1536^2 x 2048 0.94 / 0.91 / 1.02 stay in-loop)
    const bool pays_cplx = ro && ((k >= 256 && mn_ratio >= 1500.0) || (k >= 384 && mn_ratio >= 1250.0) ||
                                  (k >= 512 && mn_ratio >= 1000.0));
    const bool pays = CPLX ? pays_cplx : (pays_nt || pays_short);
    // The uncorrected modes issue a third (FP16TC) or as many (bf16x2) MFMAs per
    // element as FP16TCEC, so the same pre-pass weighs three times as much for
    // the former: it is taken for large square-ish problems only.
    // Measured (in-loop -> pre-split, TFLOP/s): FP16TC 8192^3 580 - 624 -> 930 - 940, 4096^3 586 - 706 ->
    // 852 - 870, 4096^2 x 1024 505 - 566 -> 634 - 654, 8192^2 x 512 482 - 520 -> 579 - 601, 16384^2 x 256
    // 390 - 407 -> 461 - 480, 4096^2 x 512 level; bf16x2 8192^3 320 - 377 -> 394 - 396, 4096^2 x 1024
    // 304 - 337 -> 348 - 355, 8192^2 x 512 275 - 308 -> 318 - 327, 4096^2 x 512 level except NT.
    // Complex (the 128x64 kernels): FP16TC 4096^3 560 - 678 -> 872 - 891, 2048^3 525 - 640 -> 760 - 779,
    // 8192^2 x 256 477 - 543 -> 624 - 643; bf16x2 4096^3 350 -> 375, 4096^2 x 1024 333 - 339 -> 365,
    // 4096^2 x 512 303 - 326 -> 336 - 347.
    const bool pays_tc =
        ro &&
        (CPLX ? (k >= 256 && mn_ratio >= 1000.0)
              : ((k >= 1024 && mn_ratio >= (mode == CUMPSGEMM_FP16TC ? 1500.0 : 2000.0)) ||
                 (k >= 512 && mn_ratio >= 4000.0) || (k >= 256 && mn_ratio >= 8000.0) ||
                 (mode == CUMPSGEMM_TF32TC && pays_nt_shape)));
    // (complex bf16x3, two-buffer pre-split kernel against the in-loop one, NN / TN, TFLOP/s: 4096^3 228 / 238 ->
    // 237 / 237, 3072^2 x 1024 205 / 215 -> 223 / 223, 4096^2 x 512 211 / 216 -> 230 / 226, 8192^2 x 256 197 / 205 ->
    // 219 / 218, 3072^2 x 384 189 / 199 -> 203 / 202, 2048^2 x 1024 222 / 230 -> 231 / 231, 4096^2 x 256 198 / 205 ->
    // 206 / 210; 2048^2 x 512 level: the complex rule above)
    const bool pays_b3 = CPLX ? pays_cplx : pays_bf16;
    return ch.bf16 ? (pays_b3 || always) : (ch.tc_only ? (pays_tc || always) : (pays || pays_scaled || always));
  };
  const bool mode_ok = mode == CUMPSGEMM_FP16TCEC || ch.bf16 || ch.auto_ok || ch.tc_only;
  // (CUMPSGEMM_FORCE_TILE_CLASS / _FORCE_KSPLIT pick among the in-loop kernels and keep a call off this
  // path -- except a call of the entry point that allocates nothing, which is defined to take it)
  const bool base_ok = mode_ok && !never && shape_ok && (forced || (force_cls <= 0 && force_split <= 1));
  ch.take = base_ok && worth_if(rounds_ok);
  // With a mostly empty last round the path still pays for the rounds before
  // it: the caller cuts C there (6000^2 x 2048: 332 TFLOP/s in-loop, 384 with
  // everything pre-split and a fifth round that is 40 % full).
  ch.cut = base_ok && !ch.take && !always && depth == 0 && mode != CUMPSGEMM_AUTO && ptiles > h->num_cus &&
           worth_if(true);
  // AUTO: the bf16x3 candidate gets its own (gated) pre-pass and planes behind the fp16 ones
  ch.auto_bf16 = ch.take && ch.auto_ok && pays_bf16;
  return ch;
}

// The handle's workspace only grows.  Returns the buffer, or nullptr: no memory
// or over the cap (the caller falls back to the in-loop kernels) or, with
// *failed set, the stream is broken.
void *ensure_pack_workspace(cuMpSGEMM_handle *h, uint64_t bytes, bool *failed) {
  *failed = false;
  if (h->ws_override != nullptr) return bytes <= h->ws_override_bytes ? h->ws_override : nullptr;
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(h->stream, &cap) != hipSuccess) (void)hipGetLastError();
  const bool capturing = cap != hipStreamCaptureStatusNone;
  if (h->pack_ws_bytes >= bytes && h->pack_ws != nullptr) {
    // a graph being captured now will hold this address for as long as it lives
    if (capturing) h->pack_ws_captured = true;
    return h->pack_ws;
  }
  if (bytes > tuning().max_workspace_bytes) return nullptr;
  // no allocation or synchronisation while the stream is being captured into a
  // graph: the call takes the path that needs no workspace instead
  if (capturing) return nullptr;
  // the previous workspace may still be in use by work queued on the stream
  if (hipStreamSynchronize(h->stream) != hipSuccess) {
    log_error("stream synchronisation failed before growing the pack workspace");
    *failed = true;
    return nullptr;
  }
  if (h->pack_ws != nullptr) {
    // a captured graph may replay at any time: its workspace stays until the
    // handle is destroyed
    if (h->pack_ws_captured) h->retired_ws.push_back(h->pack_ws);
    else (void)hipFree(h->pack_ws);
  }
  h->pack_ws_captured = false;
  h->pack_ws = nullptr;
  h->pack_ws_bytes = 0;
  if (hipMalloc(&h->pack_ws, bytes) != hipSuccess) {
    (void)hipGetLastError();
    h->pack_ws = nullptr;
    return nullptr;
  }
  h->pack_ws_bytes = bytes;
  return h->pack_ws;
}

// `args`: the call's arguments (scalars, C, conj flags, launch flag); `accept_*`:
// the launch-flag masks of the two AUTO candidates.
template <class T>
PreSplit run_pre_split(cuMpSGEMM_handle *h, const GemmArgs &args, bool a_kc, bool b_kc, uint64_t m,
                       uint64_t n, uint64_t k, const T *a, uint64_t lda, const T *b, uint64_t ldb,
                       uint64_t batch, cuMpSGEMM_compute_mode_t mode, uint32_t accept_bf16,
                       uint32_t accept_fp16, int force_cls, int force_split, int depth,
                       unsigned *used_id) {
  constexpr bool CPLX = std::is_same<T, hipComplex>::value;
  const PreSplitChoice ch = choose_pre_split<CPLX>(h, a_kc, b_kc, m, n, k, batch, mode, force_cls, force_split, depth);
  if (!ch.take) return PreSplit::NOT_TAKEN;
  const uint32_t mp = packed_rows(m), np = packed_rows(n);
  const uint64_t a_bytes = packed_bytes(mp, k, ch.planes), b_bytes = packed_bytes(np, k, ch.planes);
  const uint64_t a3_bytes = ch.auto_bf16 ? packed_bytes(mp, k, 3) : 0;
  const uint64_t b3_bytes = ch.auto_bf16 ? packed_bytes(np, k, 3) : 0;
  const uint64_t ws_bytes = a_bytes + b_bytes + a3_bytes + b3_bytes;
  if (mp * 64ull >= 0xffffffffull || np * 64ull >= 0xffffffffull) return PreSplit::NOT_TAKEN;
  bool failed = false;
  void *const ws = ensure_pack_workspace(h, ws_bytes, &failed);
  if (ws == nullptr) return failed ? PreSplit::FAILED : PreSplit::NOT_TAKEN;

  const float *af = reinterpret_cast<const float *>(a), *bf = reinterpret_cast<const float *>(b);
  const int *gate = ch.auto_ok ? args.launch_flag : nullptr;
  constexpr int kWalkAlways = 0, kWalkShort = 1, kWalkNever = 2, kWalkMid = 3; // K ranges of the persistent form
  // one candidate: pre-pass of both operands, then the kernel over their planes
  auto run = [&](PackKind kind, char *pa, char *pb, int bm, int bn, uint32_t accept, bool scaled,
                 auto launch_kernel, int walk_rule) -> bool {
    GemmArgs pargs = args;
    const uint32_t *max_a = nullptr, *max_b = nullptr;
    const int *sflag = nullptr;
    if (scaled) {
      max_a = &h->stats_slots[h->fused_slot_a].max_exp_bits;
      max_b = &h->stats_slots[h->fused_slot_b].max_exp_bits;
      sflag = h->flag_buffer + h->fused_flag;
      pargs.scale_max_a = max_a; // the kernel derives the inverse scaling of C from them
      pargs.scale_max_b = max_b;
      pargs.scale_flag = sflag;
    }
    launch_pack_split_pair(h->stream, PackOperand{af, a_kc, lda, (uint32_t)m, pa, mp, max_a},
                           PackOperand{bf, b_kc, ldb, (uint32_t)n, pb, np, max_b}, (uint32_t)k, kind, sflag, gate,
                           accept);
    pargs.a = pa;
    pargs.b = pb;
    pargs.lda = mp; // padded row counts of the packed operands
    pargs.ldb = np;
    pargs.k = (uint32_t)((k + 31) / 32 * 32); // zero-padded to whole K-steps
    pargs.k_chunk = pargs.k;
    pargs.tiles_m = (uint32_t)((m + bm - 1) / bm);
    pargs.tiles_n = (uint32_t)((n + bn - 1) / bn);
    pargs.batch = 1;
    pargs.atomic_out = 0;
    // Tile order: column groups of 4 tile rows keep the patch of C that an
    // XCD's 32 resident tiles cover near square, which is what its L2 reuses
    // best (the in-loop kernels keep 8); measured + 1 - 4 % over 8 for every
    // pre-split kernel, except that the fp16 one runs best with 2 from
    // K = 8192 on (12288^2 x 8192: 391 with 2, 384 with 4, 377 TFLOP/s with 8).
    // (args.raster_group != 0: set by CUMPSGEMM_RASTER_GROUP)
    if (args.raster_group == 0) pargs.raster_group = (kind == PackKind::FP16_REAL && k >= 8192) ? 2u : 4u;
    pargs.launch_flag = gate;
    pargs.flag_accept_mask = accept;
    const uint64_t total = (uint64_t)pargs.tiles_m * pargs.tiles_n;
    // Persistent workgroups that walk a list of tiles, or a workgroup per tile:
    // (real FP16TCEC / bf16x3 / bf16x2: the tile-walking form with global -> LDS loads at every K --
    // 8192^3 381 - 384 against 365 - 368 TFLOP/s, 16384^2 x 1024 374 against 353, 16384^2 x 256 297 against 262;
    // complex FP16TCEC / bf16x2: up to 32 K-steps -- 8192^2 x 384 390 against 367, 4096^2 x 512 381 against
    // 370, level from there on; FP16TC, real and complex, has its two one-tile workgroups per CU)
    bool walk = walk_rule == kWalkNever ? false
                : (walk_rule == kWalkAlways ? true
                   : (walk_rule == kWalkMid ? pargs.k / 32 <= 32 : pargs.k / 32 < 16));
    if (tuning().packed_walk >= 0) walk = tuning().packed_walk == 1;
    if (kind == PackKind::BF16X3_COMPLEX) walk = false; // (its kernel has the one-tile form only)
    if (walk && tuning().fetch_from_one_patch) pargs.raster_group |= kFetchFromOnePatch; // (profiler experiment)
    const dim3 grid = walk ? dim3((unsigned)std::min<uint64_t>(total, h->num_cus), 1, 1)
                           : dim3((unsigned)total, 1, 1);
    launch_kernel(pargs, grid, walk);
    const hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
      log_error(std::string("packed GEMM launch failed: ") + hipGetErrorString(err));
      return false;
    }
    return true;
  };

  char *pa = static_cast<char *>(ws), *pb = pa + a_bytes;
  const uint32_t accept = ch.auto_ok ? accept_fp16 : 0u;
  bool ok;
  if constexpr (CPLX) {
    if (ch.bf16) {
      ok = run(PackKind::BF16X3_COMPLEX, pa, pb, ch.bm, ch.bn, 0u, false,
               [&](const GemmArgs &g, dim3 grid, bool) { launch_packed_bf16x3_c(g, grid, h->stream); }, kWalkNever);
    } else if (ch.tc_only) {
      const bool fp16 = mode == CUMPSGEMM_FP16TC;
      ok = run(fp16 ? PackKind::FP16TC_COMPLEX : PackKind::BF16X2_COMPLEX, pa, pb, ch.bm, ch.bn, 0u, false,
               [&](const GemmArgs &g, dim3 grid, bool walk) {
                 if (fp16) launch_packed_fp16tc_c(g, grid, h->stream, walk);
                 else launch_packed_bf16x2_c(g, grid, h->stream, walk);
               }, fp16 ? kWalkNever : kWalkMid);
    } else {
      ok = run(PackKind::FP16_COMPLEX, pa, pb, ch.bm, ch.bn, accept, h->fused_scaling,
               [&](const GemmArgs &g, dim3 grid, bool walk) {
                 launch_packed_fp16tcec_c(g, grid, h->stream, walk, h->fused_scaling);
               }, kWalkMid);
    }
  } else if (ch.bf16) {
    ok = run(PackKind::BF16X3_REAL, pa, pb, ch.bm, ch.bn, accept, false,
             [&](const GemmArgs &g, dim3 grid, bool walk) { launch_packed_bf16x3_s(g, grid, h->stream, walk); },
             kWalkAlways);
  } else if (ch.tc_only) {
    const bool fp16 = mode == CUMPSGEMM_FP16TC;
    ok = run(fp16 ? PackKind::FP16TC_REAL : PackKind::BF16X2_REAL, pa, pb, ch.bm, ch.bn, 0u, false,
             [&](const GemmArgs &g, dim3 grid, bool walk) {
               if (fp16) launch_packed_fp16tc_s(g, grid, h->stream, walk);
               else launch_packed_bf16x2_s(g, grid, h->stream, walk);
             }, fp16 ? kWalkShort : kWalkAlways); // (FP16TC: two one-tile workgroups per CU from 16 K-steps on)
  } else {
    ok = run(PackKind::FP16_REAL, pa, pb, ch.bm, ch.bn, accept, h->fused_scaling,
             [&](const GemmArgs &g, dim3 grid, bool walk) {
               if (h->fused_scaling) launch_packed_scaled_fp16tcec_s(g, grid, h->stream, walk);
               else launch_packed_fp16tcec_s(g, grid, h->stream, walk);
             }, kWalkAlways);
  }
  if (!ok) return PreSplit::FAILED;
  if (used_id != nullptr) *used_id = 200u; // pre-split path
  if (!ch.auto_ok) return PreSplit::DONE;
  if (!ch.auto_bf16) return PreSplit::FP16_SERVED;
  // AUTO, the other candidate by the same path: three bf16 planes, its own accept mask
  if constexpr (!CPLX) {
    char *pa3 = pb + b_bytes, *pb3 = pa3 + a3_bytes;
    ok = run(PackKind::BF16X3_REAL, pa3, pb3, kPackedBf16BM, kPackedBf16BN, accept_bf16, false,
             [&](const GemmArgs &g, dim3 grid, bool walk) { launch_packed_bf16x3_s(g, grid, h->stream, walk); },
             kWalkAlways);
    if (!ok) return PreSplit::FAILED;
  }
  if (used_id != nullptr) *used_id = ~0u; // AUTO
  return PreSplit::DONE;
}


template <class T>
hipblasStatus_t run_gemm(cuMpSGEMM_handle *h, hipblasOperation_t op_A,
                         hipblasOperation_t op_B, uint64_t m, uint64_t n, uint64_t k,
                         const T *alpha, const T *a, uint64_t lda, uint64_t stridea,
                         const T *b, uint64_t ldb, uint64_t strideb, const T *beta, T *c,
                         uint64_t ldc, uint64_t stridec, uint64_t batch,
                         cuMpSGEMM_compute_mode_t mode, unsigned *used_id,
                         const char *label, int depth = 0) {
  constexpr bool CPLX = std::is_same<T, hipComplex>::value;
  if (h == nullptr || alpha == nullptr || beta == nullptr) return HIPBLAS_STATUS_INVALID_VALUE;
  if (m == 0 || n == 0 || batch == 0) return HIPBLAS_STATUS_SUCCESS;
  if (m > 0x7fffffffull || n > 0x7fffffffull || k > 0x7fffffffull || batch > 65535ull)
    return HIPBLAS_STATUS_INVALID_VALUE;
  const bool a_kc = (op_A != HIPBLAS_OP_N);
  const bool b_kc = (op_B == HIPBLAS_OP_N);
  if (ldc < m) return HIPBLAS_STATUS_INVALID_VALUE;
  if (k != 0 && (lda < (a_kc ? k : m) || ldb < (b_kc ? k : n))) return HIPBLAS_STATUS_INVALID_VALUE;
  // a null operand would fault on the device, not fail: refuse it here
  if (c == nullptr || (k != 0 && (a == nullptr || b == nullptr))) return HIPBLAS_STATUS_INVALID_VALUE;

  GemmArgs args{};
  args.m = (uint32_t)m;
  args.n = (uint32_t)n;
  args.k = (uint32_t)k;
  args.a = a;
  args.b = b;
  args.c = c;
  args.lda = lda;
  args.ldb = ldb;
  args.ldc = ldc;
  args.stride_a = stridea;
  args.stride_b = strideb;
  args.stride_c = stridec;
  scalar_parts<T>::get(alpha, args.alpha_re, args.alpha_im);
  scalar_parts<T>::get(beta, args.beta_re, args.beta_im);
  args.conj_a = (CPLX && op_A == HIPBLAS_OP_C) ? 1u : 0u;
  args.conj_b = (CPLX && op_B == HIPBLAS_OP_C) ? 1u : 0u;
#if CUMPSGEMM_WALK_STAMPS
  args.stamps = g_walk_stamps.load();
#endif
  args.raster_group = (uint32_t)tuning().raster_group; // experiments: tile order of the one-tile kernels

  // which kernels to launch: one for a fixed mode; for AUTO both candidates,
  // each gated on the device flag so that no host synchronisation is needed
  // (reference src/cumpsgemm.cu:305-368, src/cumpsgemm_kernel.cuh:478-489)
  struct Launch {
    Prec p;
    uint32_t accept;
  } launches[2];
  int nlaunch = 0;
  if (mode == CUMPSGEMM_AUTO) {
    launches[nlaunch++] = {Prec::BF16X3, 1u << CUMPSGEMM_TF32TCEC};
    launches[nlaunch++] = {Prec::FP16TCEC,
                           (1u << CUMPSGEMM_FP16TCEC) | (1u << CUMPSGEMM_FP16TCEC_SCALING)};
    args.launch_flag = h->flag_buffer + h->flag_enabled_id;
  } else {
    Prec p;
    if (!mode_to_prec(mode, p)) return HIPBLAS_STATUS_INVALID_VALUE;
    launches[nlaunch++] = {p, 0u};
    args.launch_flag = nullptr;
  }

  const int force_cls = tuning().force_cls;
  const int force_split = tuning().force_split; // experiments: fix the split-K factor (a power of two)
  const bool no_persist = tuning().no_persistent;

  // the two halves of a column split are timed as one call, by the outer level
  struct ProfilerPause {
    cuMpSGEMM_handle *h;
    bool was, active;
    ~ProfilerPause() { if (active) h->profiler.enabled = was; }
  } pause{h, h->profiler.enabled, depth > 0};
  if (depth > 0) h->profiler.enabled = false;
  ProfileScope prof(h, label);
  const bool beta_zero = args.beta_re == 0.0f && args.beta_im == 0.0f;

  if (k == 0) { // C = beta * C
    launch_prescale_c<CPLX>(h->stream, c, args.m, args.n, ldc, stridec, (uint32_t)batch, args.beta_re,
                            args.beta_im);
    return HIPBLAS_STATUS_SUCCESS;
  }

  // large problems: operands split once, up front (see run_pre_split)
  bool fp16_served = false;
  if (nlaunch > 0) {
    const uint32_t accept_bf16 = launches[0].accept, accept_fp16 = nlaunch > 1 ? launches[1].accept : 0u;
    switch (run_pre_split<T>(h, args, a_kc, b_kc, m, n, k, a, lda, b, ldb, batch, mode, accept_bf16,
                             accept_fp16, force_cls, force_split, depth, used_id)) {
    case PreSplit::DONE:
      return HIPBLAS_STATUS_SUCCESS;
    case PreSplit::FAILED:
      return HIPBLAS_STATUS_EXECUTION_FAILED;
    case PreSplit::FP16_SERVED:
      nlaunch = 1;        // the FP16TCEC candidate is served; bf16x3 remains
      fp16_served = true; // (and is not cut into column blocks: they would come back here)
      break;
    case PreSplit::NOT_TAKEN:
      break;
    }
  }

  // C's rows and columns are independent, so a problem can be cut in two along
  // either; both parts come back here one level down (and are not cut again).
  // depth1: the level the first part runs at (2: it takes the pre-split path).
  auto run_cut = [&](const bool by_rows, const uint64_t m1, const uint64_t n1, const int depth1) {
    if (by_rows) {
      const T *a2 = a_kc ? a + m1 * lda : a + m1; // op(A) = T: columns of A^T; else rows of A
      hipblasStatus_t st = run_gemm<T>(h, op_A, op_B, m1, n, k, alpha, a, lda, stridea, b, ldb, strideb,
                                       beta, c, ldc, stridec, 1, mode, used_id, label, depth1);
      if (st != HIPBLAS_STATUS_SUCCESS) return st;
      return run_gemm<T>(h, op_A, op_B, m - m1, n, k, alpha, a2, lda, stridea, b, ldb, strideb, beta,
                         c + m1, ldc, stridec, 1, mode, nullptr, label, 1);
    }
    const T *b2 = b_kc ? b + n1 * ldb : b + n1; // op(B) = N: columns of B; else rows of B^T
    hipblasStatus_t st = run_gemm<T>(h, op_A, op_B, m, n1, k, alpha, a, lda, stridea, b, ldb, strideb,
                                     beta, c, ldc, stridec, 1, mode, used_id, label, depth1);
    if (st != HIPBLAS_STATUS_SUCCESS) return st;
    return run_gemm<T>(h, op_A, op_B, m, n - n1, k, alpha, a, lda, stridea, b2, ldb, strideb, beta,
                       c + n1 * ldc, ldc, stridec, 1, mode, nullptr, label, 1);
  };

  // The pre-split path stepped aside only because its last round of CU slots
  // would be mostly empty: cut C where its whole rounds end.  The first part
  // takes the path, the rest is planned on its own (in-loop -> cut, TFLOP/s:
  // 6000^2 x 2048 306 -> 360, 4200^3 303 -> 335).
  if (batch == 1 && depth == 0 && !fp16_served && !tuning().no_column_split) {
    const PreSplitChoice ch =
        choose_pre_split<CPLX>(h, a_kc, b_kc, m, n, k, batch, mode, force_cls, force_split, depth);
    if (ch.cut) {
      const uint64_t tm = (m + ch.bm - 1) / ch.bm, tn = (n + ch.bn - 1) / ch.bn;
      const uint64_t whole = (tm * tn / h->num_cus) * h->num_cus; // tiles of the whole rounds
      const uint64_t cols1 = whole / tm, rows1 = whole / tn;      // tile columns / rows that fit in them
      const bool by_rows = rows1 * tn > cols1 * tm;               // the cut that keeps more of them
      if (by_rows && rows1 >= 1 && rows1 < tm) return run_cut(true, rows1 * (uint64_t)ch.bm, 0, 2);
      if (!by_rows && cols1 >= 1 && cols1 < tn) return run_cut(false, 0, cols1 * (uint64_t)ch.bn, 2);
    }
  }

  // AUTO launches two gated kernels that must agree on how C is prepared, so
  // the split-K decision is taken once, from the first candidate.
  Plan plan0 = make_plan(h, launches[0].p, CPLX, a_kc, b_kc, m, n, k, batch, force_cls, force_split);
  const bool split = plan0.ksplit > 1;

  // A tile count just above a multiple of the chip's CU slots leaves most CUs
  // idle for the last round.  C's columns are independent, so such a problem is
  // cut in two: a first part whose tiles fill whole rounds, and the remaining
  // columns, planned on their own (typically with K split to fill the chip).
  if (!split && batch == 1 && depth == 0 && !fp16_served && k >= 256 &&
      !tuning().no_column_split) {
    // (C's rows are independent as well: the cut that leaves the cheaper pair of
    // problems wins -- which one that is depends on the tile's aspect ratio)
    const KernelEntry *e0 = plan0.entry;
    const uint64_t slots = (uint64_t)h->num_cus * resident_groups(e0);
    const uint64_t tiles = (uint64_t)plan0.tiles_m * plan0.tiles_n;
    const uint64_t full = tiles / slots;
    const uint64_t cols1 = (full * slots) / plan0.tiles_m; // tile columns of the first part
    const uint64_t rows1 = (full * slots) / plan0.tiles_n; // or its tile rows
    const double extra_launch = 3.0 * 256.0 * 128.0;
    auto cost_of = [&](uint64_t mm, uint64_t nn) {
      return make_plan(h, launches[0].p, CPLX, a_kc, b_kc, mm, nn, k, 1, force_cls, force_split).cost;
    };
    double cost_cols = -1.0, cost_rows = -1.0;
    const uint64_t n1 = cols1 * (uint64_t)e0->bn, m1 = rows1 * (uint64_t)e0->bm;
    if (full >= 1 && tiles % slots != 0) {
      if (cols1 >= 1 && cols1 < plan0.tiles_n) cost_cols = cost_of(m, n1) + cost_of(m, n - n1) + extra_launch;
      if (rows1 >= 1 && rows1 < plan0.tiles_m) cost_rows = cost_of(m1, n) + cost_of(m - m1, n) + extra_launch;
    }
    const bool by_rows = cost_rows >= 0.0 && (cost_cols < 0.0 || cost_rows < cost_cols);
    const double cost_cut = by_rows ? cost_rows : cost_cols;
    // How far below the uncut plan the model must price the two parts.  Measured
    // against the model on 15 shapes per kind with the cut forced and forbidden
    // (ratio of the two times): real kernels run 0.00 - 0.08 above the model's
    // ratio, complex FP16TCEC within 0.03 of it, and complex bf16x3 -- whose
    // large tile is the one kernel of a table that does not walk its tiles --
    // 0.15 - 0.23 below it (1536^3: model 0.94, measured 0.73; 1600^2 x 800: 1.09, 0.91;
    // 1920^2 x 384: 1.21, 1.03).
    const int cut_percent = tuning().cut_percent > 0
                                ? tuning().cut_percent
                                : (CPLX ? (launches[0].p == Prec::BF16X3 ? 110 : 96) : 93);
    if (cost_cut >= 0.0 && cost_cut < 0.01 * cut_percent * plan0.cost) return run_cut(by_rows, m1, n1, 1);
  }

  if (split) {
    launch_prescale_c<CPLX>(h->stream, c, args.m, args.n, ldc, stridec, (uint32_t)batch, args.beta_re,
                            args.beta_im);
  }
  (void)beta_zero;

  for (int i = 0; i < nlaunch; i++) {
    Plan plan = (i == 0) ? plan0
                         : make_plan(h, launches[i].p, CPLX, a_kc, b_kc, m, n, k, batch, force_cls, force_split);
    if (split) { // same K partition for every candidate
      plan.ksplit = plan0.ksplit;
      plan.k_chunk = plan0.k_chunk;
    } else {
      plan.ksplit = 1;
      plan.k_chunk = (unsigned)k;
    }
    args.tiles_m = plan.tiles_m;
    args.tiles_n = plan.tiles_n;
    args.batch = (uint32_t)batch;
    args.k_chunk = plan.k_chunk;
    args.atomic_out = split ? 1u : 0u;
    args.flag_accept_mask = launches[i].accept;
    const KernelEntry *e = plan.entry;
    auto launch_plain = e->launch;
    auto launch_walk = e->launch_persistent;
    if (h->fused_scaling && launches[i].p == Prec::FP16TCEC) {
      launch_plain = e->launch_scaled;
      launch_walk = e->launch_scaled_persistent;
      args.scale_max_a = &h->stats_slots[h->fused_slot_a].max_exp_bits;
      args.scale_max_b = &h->stats_slots[h->fused_slot_b].max_exp_bits;
      args.scale_flag = h->flag_buffer + h->fused_flag;
    }
    if (launch_walk != nullptr && !no_persist &&
        persistent_ok<T>(e, a_kc, b_kc, m, n, k, plan, lda, ldb, batch,
                         launch_walk == e->launch_scaled_persistent)) {
      const uint64_t slots = (uint64_t)h->num_cus * resident_groups(e);
      const uint64_t total = (uint64_t)plan.tiles_m * plan.tiles_n * batch;
      // A launch that keeps every CU busy to its end runs against the power limit
      // and takes the instance on 16x16x32 MFMAs, where the table has one (not
      // with a forced class: the test switches compare forms bit for bit).
      const uint64_t units = total * plan.ksplit, last = units % slots;
      // (measured with and without, NN / TN / TT: 256^3 x 512 1.13 / 1.08 / 1.08, 1024^3 x 8 1.06 / 1.07 / 1.05,
      // 2048^2 x 1024 x 2 1.05 / 1.07 / 1.05, 4096^2 x 384 1.03 / 1.05 / 1.03, 512^3 x 64 1.03 / 1.03 / 1.02;
      // 3584^2 x 1024, whose last round fills 53 % of the CUs: 0.98 / 1.01 / 0.98)
      if (units >= slots && (last == 0 || last >= slots * 3 / 4) && force_cls < 0 && !tuning().no_edge16_twin) {
        if (launch_walk == e->launch_scaled_persistent && e->launch_scaled_persistent_edge16 != nullptr)
          launch_walk = e->launch_scaled_persistent_edge16;
        else if (launch_walk == e->launch_persistent && e->launch_persistent_edge16 != nullptr)
          launch_walk = e->launch_persistent_edge16;
      }
      const dim3 grid((unsigned)std::min(total, slots), 1, plan.ksplit);
      launch_walk(args, grid, h->stream);
    } else {
      const dim3 grid(plan.tiles_m * plan.tiles_n, (unsigned)batch, plan.ksplit);
      // At most one small workgroup per CU: its four waves, one per SIMD, are
      // bound by the latency of their own chain of LDS reads, MFMAs and staging,
      // so the form with two wave groups (a K-slice of every step each) is
      // launched -- where it was measured faster: an operand K-contiguous and a
      // mode with correction terms or bf16 planes (1024^3, plain -> two groups,
      // us: FP16TCEC NN 19.3 -> 16.4, TN 16.2 -> 13.8, TT 18.6 -> 16.1, bf16x3 NN
      // 28.1 -> 21.5, bf16x2 NN 19.7 -> 16.5; complex FP16TCEC NN 38.6 -> 34.5,
      // bf16x2 38.0 -> 33.5; FP16TC level or slower; op(A) = N with op(B) = T level).
      const uint64_t groups = (uint64_t)grid.x * grid.y * grid.z;
      auto launch_groups = launch_plain == e->launch_scaled ? e->launch_scaled_kslices : e->launch_kslices;
      if (launch_groups != nullptr && groups <= (uint64_t)h->num_cus && (a_kc || b_kc) &&
          launches[i].p != Prec::FP16TC && !tuning().no_kslices) {
        launch_groups(args, grid, h->stream);
      } else {
        launch_plain(args, grid, h->stream);
      }
    }
    if (used_id != nullptr) {
      *used_id = (mode == CUMPSGEMM_AUTO) ? ~0u : (unsigned)plan.cls + (split ? 100u : 0u);
    }
  }
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    log_error(std::string("GEMM launch failed: ") + hipGetErrorString(err));
    return HIPBLAS_STATUS_EXECUTION_FAILED;
  }
  return HIPBLAS_STATUS_SUCCESS;
}
} // namespace
} // namespace cumpsgemm_amd

using namespace cumpsgemm_amd;

template <class T>
hipblasStatus_t cumpsgemm::gemm(cuMpSGEMM_handle_t handle, hipblasOperation_t op_A,
                                hipblasOperation_t op_B, uint64_t m, uint64_t n, uint64_t k,
                                const T *alpha, const T *a_dmem_ptr, uint64_t lda,
                                const T *b_dmem_ptr, uint64_t ldb, const T *beta,
                                T *c_dmem_ptr, uint64_t ldc,
                                cuMpSGEMM_compute_mode_t compute_mode,
                                unsigned *used_kernel_module_id) {
  return run_gemm<T>(handle, op_A, op_B, m, n, k, alpha, a_dmem_ptr, lda, 0, b_dmem_ptr, ldb, 0,
                     beta, c_dmem_ptr, ldc, 0, 1, compute_mode, used_kernel_module_id,
                     "gemm_kernel");
}

template <class T>
hipblasStatus_t cumpsgemm::gemm_stridedBatch(
    cuMpSGEMM_handle_t handle, hipblasOperation_t op_A, hipblasOperation_t op_B, uint64_t m,
    uint64_t n, uint64_t k, const T *alpha, const T *a_dmem_ptr, uint64_t lda, uint64_t stridea,
    const T *b_dmem_ptr, uint64_t ldb, uint64_t strideb, const T *beta, T *c_dmem_ptr,
    uint64_t ldc, uint64_t stridec, uint64_t batch_count, cuMpSGEMM_compute_mode_t compute_mode,
    unsigned *used_kernel_module_id) {
  // A few large matrices: each is worth the pre-split path on its own (which
  // handles one matrix at a time), so they are issued one by one, like the
  // reference does for large batches (src/cumpsgemm.cu:431-439).
  if (handle != nullptr && batch_count > 1 && batch_count <= 1024 && m <= 0x7fffffffull && n <= 0x7fffffffull &&
      k <= 0x7fffffffull) {
    constexpr bool CPLX = std::is_same<T, hipComplex>::value;
    const int force_cls = tuning().force_cls, force_split = tuning().force_split;
    const PreSplitChoice ch = choose_pre_split<CPLX>(handle, op_A != HIPBLAS_OP_N, op_B == HIPBLAS_OP_N, m, n, k, 1,
                                                     compute_mode, force_cls, force_split, 0);
    if (ch.take) {
      hipblasStatus_t st1 = HIPBLAS_STATUS_SUCCESS;
      for (uint64_t i = 0; i < batch_count && st1 == HIPBLAS_STATUS_SUCCESS; i++) {
        st1 = run_gemm<T>(handle, op_A, op_B, m, n, k, alpha, a_dmem_ptr + i * stridea, lda, 0,
                          b_dmem_ptr + i * strideb, ldb, 0, beta, c_dmem_ptr + i * stridec, ldc, 0, 1,
                          compute_mode, used_kernel_module_id, "batched_gemm_kernel");
      }
      return st1;
    }
  }
  // batches beyond the grid's y limit are issued in slices
  uint64_t done = 0;
  hipblasStatus_t st = HIPBLAS_STATUS_SUCCESS;
  while (done < batch_count && st == HIPBLAS_STATUS_SUCCESS) {
    const uint64_t nb = std::min<uint64_t>(batch_count - done, 65535);
    st = run_gemm<T>(handle, op_A, op_B, m, n, k, alpha, a_dmem_ptr + done * stridea, lda,
                     stridea, b_dmem_ptr + done * strideb, ldb, strideb, beta,
                     c_dmem_ptr + done * stridec, ldc, stridec, nb, compute_mode,
                     used_kernel_module_id, "batched_gemm_kernel");
    done += nb;
  }
  return st;
}

template hipblasStatus_t cumpsgemm::gemm<float>(cuMpSGEMM_handle_t, hipblasOperation_t,
                                                hipblasOperation_t, uint64_t, uint64_t, uint64_t,
                                                const float *, const float *, uint64_t,
                                                const float *, uint64_t, const float *, float *,
                                                uint64_t, cuMpSGEMM_compute_mode_t, unsigned *);
template hipblasStatus_t cumpsgemm::gemm<hipComplex>(
    cuMpSGEMM_handle_t, hipblasOperation_t, hipblasOperation_t, uint64_t, uint64_t, uint64_t,
    const hipComplex *, const hipComplex *, uint64_t, const hipComplex *, uint64_t,
    const hipComplex *, hipComplex *, uint64_t, cuMpSGEMM_compute_mode_t, unsigned *);
template hipblasStatus_t cumpsgemm::gemm_stridedBatch<float>(
    cuMpSGEMM_handle_t, hipblasOperation_t, hipblasOperation_t, uint64_t, uint64_t, uint64_t,
    const float *, const float *, uint64_t, uint64_t, const float *, uint64_t, uint64_t,
    const float *, float *, uint64_t, uint64_t, uint64_t, cuMpSGEMM_compute_mode_t, unsigned *);
template hipblasStatus_t cumpsgemm::gemm_stridedBatch<hipComplex>(
    cuMpSGEMM_handle_t, hipblasOperation_t, hipblasOperation_t, uint64_t, uint64_t, uint64_t,
    const hipComplex *, const hipComplex *, uint64_t, uint64_t, const hipComplex *, uint64_t,
    uint64_t, const hipComplex *, hipComplex *, uint64_t, uint64_t, uint64_t,
    cuMpSGEMM_compute_mode_t, unsigned *);

extern "C" {

hipblasStatus_t cuMpSGEMM_create(cuMpSGEMM_handle_t *handle) {
  if (handle == nullptr) return HIPBLAS_STATUS_INVALID_VALUE;
  cuMpSGEMM_handle *h = new (std::nothrow) cuMpSGEMM_handle;
  if (h == nullptr) return HIPBLAS_STATUS_ALLOC_FAILED;
  *handle = nullptr;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
    delete h;
    return HIPBLAS_STATUS_NOT_INITIALIZED;
  }
  h->device = dev;
  h->num_cus = (unsigned)cus;
  (void)scratch_address(dev); // set-up for cuMpSGEMM_sgemm_no_alloc, once per device
  bool ok = true;
  ok = ok && hipMalloc(&h->stats_slots, sizeof(StatsSlot) * h->stats_ring_length) == hipSuccess;
  ok = ok && hipMalloc(&h->stats_partials, sizeof(StatsPartial) * kMaxStatsBlocks) == hipSuccess;
  ok = ok && hipMalloc(&h->stats_ticket, 3 * sizeof(unsigned)) == hipSuccess;
  ok = ok && hipMalloc(&h->flag_buffer, sizeof(int) * h->flag_ring_length) == hipSuccess;
  ok = ok && hipHostMalloc(&h->host_scratch, sizeof(unsigned long long) * 4, hipHostMallocDefault) ==
                 hipSuccess;
  if (!ok) {
    cuMpSGEMM_destroy(h);
    return HIPBLAS_STATUS_ALLOC_FAILED;
  }
  ok = ok && hipMemsetAsync(h->stats_slots, 0, sizeof(StatsSlot) * h->stats_ring_length, nullptr) == hipSuccess;
  ok = ok && hipMemsetAsync(h->flag_buffer, 0, sizeof(int) * h->flag_ring_length, nullptr) == hipSuccess;
  hipLaunchKernelGGL(init_rings_kernel, dim3(1), dim3(1), 0, nullptr, h->stats_slots,
                     h->flag_buffer, h->stats_ticket);
  ok = ok && hipStreamSynchronize(nullptr) == hipSuccess;
  if (!ok) {
    cuMpSGEMM_destroy(h);
    return HIPBLAS_STATUS_INTERNAL_ERROR;
  }
  *handle = h;
  return HIPBLAS_STATUS_SUCCESS;
}

hipblasStatus_t cuMpSGEMM_destroy(cuMpSGEMM_handle_t handle) {
  if (handle == nullptr) return HIPBLAS_STATUS_SUCCESS;
  (void)hipFree(handle->stats_slots);
  (void)hipFree(handle->stats_partials);
  (void)hipFree(handle->stats_ticket);
  (void)hipFree(handle->flag_buffer);
  if (handle->pack_ws != nullptr) (void)hipFree(handle->pack_ws);
  for (void *p : handle->retired_ws) (void)hipFree(p);
  if (handle->order_event != nullptr) (void)hipEventDestroy(handle->order_event);
  if (handle->host_scratch) (void)hipHostFree(handle->host_scratch);
  delete handle;
  return HIPBLAS_STATUS_SUCCESS;
}

hipblasStatus_t cuMpSGEMM_set_stream(cuMpSGEMM_handle_t handle, hipStream_t stream) {
  if (handle == nullptr) return HIPBLAS_STATUS_INVALID_VALUE;
  if (stream != handle->stream) {
    // order the new stream behind the handle's work on the old one (a stream
    // under graph capture is left alone: its work runs when the graph does)
    hipStreamCaptureStatus old_cap = hipStreamCaptureStatusNone, new_cap = hipStreamCaptureStatusNone;
    (void)hipStreamIsCapturing(handle->stream, &old_cap);
    (void)hipStreamIsCapturing(stream, &new_cap);
    if (old_cap == hipStreamCaptureStatusNone && new_cap == hipStreamCaptureStatusNone) {
      if (handle->order_event == nullptr &&
          hipEventCreateWithFlags(&handle->order_event, hipEventDisableTiming) != hipSuccess) {
        handle->order_event = nullptr;
        (void)hipGetLastError();
      }
      if (handle->order_event != nullptr) {
        if (hipEventRecord(handle->order_event, handle->stream) != hipSuccess ||
            hipStreamWaitEvent(stream, handle->order_event, 0) != hipSuccess) {
          (void)hipGetLastError();
          (void)hipStreamSynchronize(handle->stream); // the blunt way
        }
      } else {
        (void)hipStreamSynchronize(handle->stream);
      }
    }
    (void)hipGetLastError();
  }
  handle->stream = stream;
  return HIPBLAS_STATUS_SUCCESS;
}

const char *cuMpSGEMM_get_compute_mode_string(cuMpSGEMM_compute_mode_t mode) {
  static const char *const names[] = {
      "CUBLAS",        "FP16TCEC",      "TF32TCEC", "FP16TC", "TF32TC",    "CUBLAS_SIMT",
      "CUBLAS_FP16TC", "CUBLAS_TF32TC", "DRY_RUN",  "AUTO",   "UNDEFINED", "FP16TCEC_SCALING",
      "FP32_SIMT"};
  const int i = (int)mode;
  return (i >= 0 && i <= 12) ? names[i] : "Unknown";
}

hipblasStatus_t cuMpSGEMM_sgemm(cuMpSGEMM_handle_t handle, hipblasOperation_t op_A,
                                hipblasOperation_t op_B, uint64_t m, uint64_t n, uint64_t k,
                                const float *alpha, const float *a_dmem_ptr, uint64_t lda,
                                const float *b_dmem_ptr, uint64_t ldb, const float *beta,
                                float *c_dmem_ptr, uint64_t ldc,
                                cuMpSGEMM_compute_mode_t compute_mode) {
  return cumpsgemm::gemm<float>(handle, op_A, op_B, m, n, k, alpha, a_dmem_ptr, lda, b_dmem_ptr,
                                ldb, beta, c_dmem_ptr, ldc, compute_mode);
}

hipblasStatus_t cuMpSGEMM_cgemm(cuMpSGEMM_handle_t handle, hipblasOperation_t op_A,
                                hipblasOperation_t op_B, uint64_t m, uint64_t n, uint64_t k,
                                const hipComplex *alpha, const hipComplex *a_dmem_ptr,
                                uint64_t lda, const hipComplex *b_dmem_ptr, uint64_t ldb,
                                const hipComplex *beta, hipComplex *c_dmem_ptr, uint64_t ldc,
                                cuMpSGEMM_compute_mode_t compute_mode) {
  return cumpsgemm::gemm<hipComplex>(handle, op_A, op_B, m, n, k, alpha, a_dmem_ptr, lda,
                                     b_dmem_ptr, ldb, beta, c_dmem_ptr, ldc, compute_mode);
}

hipblasStatus_t cuMpSGEMM_sgemm_strided_batch(
    cuMpSGEMM_handle_t handle, hipblasOperation_t op_A, hipblasOperation_t op_B, uint64_t m,
    uint64_t n, uint64_t k, const float *alpha, const float *a_dmem_ptr, uint64_t lda,
    uint64_t stridea, const float *b_dmem_ptr, uint64_t ldb, uint64_t strideb, const float *beta,
    float *c_dmem_ptr, uint64_t ldc, uint64_t stridec, uint64_t batch_count,
    cuMpSGEMM_compute_mode_t compute_mode) {
  return cumpsgemm::gemm_stridedBatch<float>(handle, op_A, op_B, m, n, k, alpha, a_dmem_ptr, lda,
                                             stridea, b_dmem_ptr, ldb, strideb, beta, c_dmem_ptr,
                                             ldc, stridec, batch_count, compute_mode);
}

hipblasStatus_t cuMpSGEMM_cgemm_strided_batch(
    cuMpSGEMM_handle_t handle, hipblasOperation_t op_A, hipblasOperation_t op_B, uint64_t m,
    uint64_t n, uint64_t k, const hipComplex *alpha, const hipComplex *a_dmem_ptr, uint64_t lda,
    uint64_t stridea, const hipComplex *b_dmem_ptr, uint64_t ldb, uint64_t strideb,
    const hipComplex *beta, hipComplex *c_dmem_ptr, uint64_t ldc, uint64_t stridec,
    uint64_t batch_count, cuMpSGEMM_compute_mode_t compute_mode) {
  return cumpsgemm::gemm_stridedBatch<hipComplex>(handle, op_A, op_B, m, n, k, alpha, a_dmem_ptr,
                                                  lda, stridea, b_dmem_ptr, ldb, strideb, beta,
                                                  c_dmem_ptr, ldc, stridec, batch_count,
                                                  compute_mode);
}

// ---- extension entry points (cumpsgemm_ext.h) -------------------------------
hipblasStatus_t cuMpSGEMM_sgemm_ex(cuMpSGEMM_handle_t handle, hipblasOperation_t op_A,
                                   hipblasOperation_t op_B, uint64_t m, uint64_t n, uint64_t k,
                                   const float *alpha, const float *a, uint64_t lda,
                                   const float *b, uint64_t ldb, const float *beta, float *c,
                                   uint64_t ldc, cuMpSGEMM_compute_mode_t mode,
                                   unsigned *used_kernel_module_id) {
  return cumpsgemm::gemm<float>(handle, op_A, op_B, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc,
                                mode, used_kernel_module_id);
}
hipblasStatus_t cuMpSGEMM_cgemm_ex(cuMpSGEMM_handle_t handle, hipblasOperation_t op_A,
                                   hipblasOperation_t op_B, uint64_t m, uint64_t n, uint64_t k,
                                   const hipComplex *alpha, const hipComplex *a, uint64_t lda,
                                   const hipComplex *b, uint64_t ldb, const hipComplex *beta,
                                   hipComplex *c, uint64_t ldc, cuMpSGEMM_compute_mode_t mode,
                                   unsigned *used_kernel_module_id) {
  return cumpsgemm::gemm<hipComplex>(handle, op_A, op_B, m, n, k, alpha, a, lda, b, ldb, beta, c,
                                     ldc, mode, used_kernel_module_id);
}

hipblasStatus_t cuMpSGEMM_sgemm_no_alloc(cuMpSGEMM_handle_t handle, hipblasOperation_t op_A,
                                         hipblasOperation_t op_B, uint64_t m, uint64_t n, uint64_t k,
                                         const float *alpha, const float *a, uint64_t lda, const float *b,
                                         uint64_t ldb, const float *beta, float *c, uint64_t ldc,
                                         cuMpSGEMM_compute_mode_t mode) {
  if (handle == nullptr) return HIPBLAS_STATUS_INVALID_VALUE;
  if (mode != CUMPSGEMM_FP16TCEC && mode != CUMPSGEMM_TF32TCEC) {
    log_error("cuMpSGEMM_sgemm_no_alloc serves FP16TCEC and TF32TCEC only");
    return HIPBLAS_STATUS_INVALID_VALUE;
  }
  if (m == 0 || n == 0) return HIPBLAS_STATUS_SUCCESS;
  if (k < 128 || m > 0x7fffffffull || n > 0x7fffffffull || k > 0x7fffffffull) {
    log_error("cuMpSGEMM_sgemm_no_alloc needs 128 <= k and sizes below 2^31");
    return HIPBLAS_STATUS_INVALID_VALUE;
  }
  const unsigned planes = mode == CUMPSGEMM_TF32TCEC ? 3u : 2u;
  const unsigned long long need =
      packed_bytes(packed_rows(m), k, planes) + packed_bytes(packed_rows(n), k, planes);
  if (need > kStaticScratchBytes) {
    log_error("cuMpSGEMM_sgemm_no_alloc: the split operands need " + std::to_string(need) +
              " bytes, the static scratch holds " + std::to_string(kStaticScratchBytes) +
              " ((m + n rounded up to 256) * (k rounded up to 32) * " + std::to_string(2 * planes) + " bytes)");
    return HIPBLAS_STATUS_INVALID_VALUE;
  }
  void *const ptr = scratch_address(handle->device);
  if (ptr == nullptr) return HIPBLAS_STATUS_NOT_INITIALIZED;
  handle->ws_override = ptr;
  handle->ws_override_bytes = kStaticScratchBytes;
  const hipblasStatus_t st = cumpsgemm::gemm<float>(handle, op_A, op_B, m, n, k, alpha, a, lda, b, ldb, beta, c,
                                                    ldc, mode, nullptr);
  handle->ws_override = nullptr;
  handle->ws_override_bytes = 0;
  return st;
}

hipblasStatus_t cuMpSGEMM_set_walk_stamp_buffer(void *device_buffer) {
#if CUMPSGEMM_WALK_STAMPS
  g_walk_stamps.store(static_cast<unsigned long long *>(device_buffer));
  return HIPBLAS_STATUS_SUCCESS;
#else
  (void)device_buffer;
  return HIPBLAS_STATUS_NOT_SUPPORTED;
#endif
}

size_t cuMpSGEMM_get_static_scratch_size(void) { return (size_t)kStaticScratchBytes; }

size_t cuMpSGEMM_get_workspace_size(cuMpSGEMM_handle_t handle) {
  return handle != nullptr ? (size_t)handle->pack_ws_bytes : 0;
}
const void *cuMpSGEMM_get_workspace_pointer(cuMpSGEMM_handle_t handle) {
  return handle != nullptr ? handle->pack_ws : nullptr;
}
void cuMpSGEMM_reload_tuning_env(void) {
  std::lock_guard<std::mutex> lock(g_tuning_mutex);
  g_tuning.store(new Tuning(read_tuning_env()), std::memory_order_release);
}

int cuMpSGEMM_describe_tile_config(int compute_mode, int is_complex, int op_A, int op_B,
                                   int tile_class, char *buf, size_t buf_len) {
  Prec p;
  if (!mode_to_prec((cuMpSGEMM_compute_mode_t)compute_mode, p) || tile_class < 0 ||
      tile_class >= kNumTileClasses || buf == nullptr || buf_len == 0)
    return -1;
  const KernelEntry *e = lookup_kernel(p, is_complex != 0, op_A != HIPBLAS_OP_N,
                                       op_B == HIPBLAS_OP_N, tile_class);
  std::snprintf(buf, buf_len, "%s threads=%d lds=%d occ=%d", e->name, e->threads, e->lds_bytes,
                e->occ);
  return 0;
}
} // extern "C"
