// libkeops_hip: hiprtc JIT, module loading, shape/range preprocessing and kernel launches for the
// MI355X map-reduce backend.  C ABI declared in include/keops_hip.h.
//
// Host-side counterpart of the reference's nvrtc binder:
//   keopscore/keopscore/binders/nvrtc/nvrtc_jit.cpp:38-136      -> keops_hip_compile
//   keopscore/keopscore/binders/nvrtc/keops_nvrtc.cpp:328-388   -> keops_hip_module_create/destroy
//   keopscore/keopscore/binders/nvrtc/keops_nvrtc.cpp:390-643   -> keops_hip_launch
//   keopscore/keopscore/include/Sizes.h, Ranges.h, ranges_utils.h -> ShapeTable / RangeSet below
#include "../../include/keops_hip.h"
#include "keops_static.h"

#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <map>
#include <mutex>
#include <numeric>
#include <sstream>
#include <string>
#include <vector>

#include <unistd.h>

namespace {

thread_local std::string g_last_error;

int fail(int code, const std::string& msg) {
  g_last_error = "[KeOps-HIP] " + msg;
  return code == 0 ? -1 : code;
}

#define HIP_TRY(expr)                                                                          \
  do {                                                                                         \
    hipError_t e_ = (expr);                                                                    \
    if (e_ != hipSuccess)                                                                      \
      return fail((int)e_, std::string(#expr) + " failed: " + hipGetErrorString(e_));          \
  } while (0)

// ---- embedded kernel templates (generated from csrc/kernels/*.h at build time) -------------
struct EmbeddedHeader {
  const char* name;
  const char* text;
};
#include "kernels_embedded.inc"

// ---- module file -----------------------------------------------------------------------------

std::string collect_meta(const char* src) {
  std::istringstream in(src);
  std::string line, meta;
  while (std::getline(in, line)) {
    if (line.rfind("//@keops ", 0) == 0) meta += line.substr(9) + "\n";
  }
  return meta;
}

std::map<std::string, std::string> parse_meta(const std::string& meta) {
  std::map<std::string, std::string> kv;
  std::istringstream in(meta);
  std::string tok;
  while (in >> tok) {
    size_t eq = tok.find('=');
    if (eq != std::string::npos) kv[tok.substr(0, eq)] = tok.substr(eq + 1);
  }
  return kv;
}

std::string target_arch(int device_id) {
  int n = 0;
  if (hipGetDeviceCount(&n) == hipSuccess && n > 0) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device_id >= 0 && device_id < n ? device_id : 0) == hipSuccess) {
      std::string a = prop.gcnArchName;  // e.g. "gfx950:sramecc+:xnack-"
      return a.substr(0, a.find(':'));
    }
  } else {
    (void)hipGetLastError();
  }
  const char* env = std::getenv("KEOPS_HIP_ARCH");
  return env && *env ? env : "gfx950";
}

// ---- shape table: Sizes.h ----------------------------------------------------------------------

struct ShapeTable {
  int nargs = 0, nbatchdims = 0;
  int64_t M = 0, N = 0, nbatches = 1;
  std::vector<int64_t> shapes;  // (nargs+1) x (nbatchdims+3): [batch.., M, N, D]

  int64_t* row(int k) { return shapes.data() + (size_t)k * (nbatchdims + 3); }
  const int64_t* row(int k) const { return shapes.data() + (size_t)k * (nbatchdims + 3); }

  // Mirrors Sizes<TYPE>::Sizes / fill_shape / check_ranges (Sizes.h:86-150,176-330) with the
  // checks enabled: a mismatch is an error instead of undefined behaviour.
  int build(int nargs_, const std::vector<std::vector<int64_t>>& argshapes, int64_t nx, int64_t ny,
            int64_t dimout, const std::vector<int>& indsI, const std::vector<int>& indsJ,
            const std::vector<int>& indsP, const std::vector<int64_t>& dimsX,
            const std::vector<int64_t>& dimsY, const std::vector<int64_t>& dimsP, std::string& err) {
    nargs = nargs_;
    int posI = indsI.empty() ? -1 : *std::min_element(indsI.begin(), indsI.end());
    int posJ = indsJ.empty() ? -1 : *std::min_element(indsJ.begin(), indsJ.end());
    int pos = std::max(posI, posJ);
    nbatchdims = pos > -1 ? (int)argshapes[pos].size() - 2 : 0;
    if (nbatchdims < 0) {
      err = "argument " + std::to_string(pos) + " must have at least 2 dimensions";
      return -2;
    }
    const int W = nbatchdims + 3;
    shapes.assign((size_t)(nargs + 1) * W, 1);
    shapes[nbatchdims] = nx;
    shapes[nbatchdims + 1] = ny;
    shapes[nbatchdims + 2] = dimout;

    auto batch = [&](int i, const std::vector<int64_t>& shp) -> bool {
      int64_t* r = row(i + 1);
      for (int b = 0; b < nbatchdims; b++) {
        r[b] = shp[b];
        if (r[b] != 1) {
          if (shapes[b] == 1) shapes[b] = r[b];
          else if (shapes[b] != r[b]) {
            err = "batch dimension " + std::to_string(b) + " of argument " + std::to_string(i) + " is " +
                  std::to_string(r[b]) + " but was " + std::to_string(shapes[b]) + " or 1 in previous arguments";
            return false;
          }
        }
      }
      return true;
    };
    auto check_var = [&](int i, int64_t dim, int cat, int64_t len) -> bool {
      if (i < 0 || i >= nargs) { err = "variable index " + std::to_string(i) + " out of range"; return false; }
      const int want = cat == 2 ? nbatchdims + 1 : nbatchdims + 2;
      // an argument with fewer leading dimensions is broadcast over the missing batch dimensions
      std::vector<int64_t> shp = argshapes[i];
      if ((int)shp.size() < want && (int)shp.size() >= (cat == 2 ? 1 : 2)) shp.insert(shp.begin(), want - shp.size(), 1);
      if ((int)shp.size() != want) {
        err = "argument " + std::to_string(i) + " has " + std::to_string(shp.size()) + " dimensions, expected " +
              std::to_string(want);
        return false;
      }
      if (!batch(i, shp)) return false;
      int64_t* r = row(i + 1);
      if (cat == 2) {
        r[nbatchdims + 2] = shp[nbatchdims];
      } else {
        r[nbatchdims + cat] = shp[nbatchdims];
        r[nbatchdims + 2] = shp[nbatchdims + 1];
        if (shp[nbatchdims] != len) {
          err = "argument " + std::to_string(i) + " has " + std::to_string(shp[nbatchdims]) + " rows, expected " +
                std::to_string(len);
          return false;
        }
      }
      if (r[nbatchdims + 2] != dim) {
        err = "argument " + std::to_string(i) + " has vector size " + std::to_string(r[nbatchdims + 2]) +
              " but the formula expects " + std::to_string(dim);
        return false;
      }
      return true;
    };
    for (size_t k = 0; k < indsI.size(); k++) if (!check_var(indsI[k], dimsX[k], 0, nx)) return -2;
    for (size_t k = 0; k < indsJ.size(); k++) if (!check_var(indsJ[k], dimsY[k], 1, ny)) return -2;
    for (size_t k = 0; k < indsP.size(); k++) if (!check_var(indsP[k], dimsP[k], 2, 0)) return -2;
    M = shapes[nbatchdims];
    N = shapes[nbatchdims + 1];
    nbatches = 1;
    for (int b = 0; b < nbatchdims; b++) nbatches *= shapes[b];
    return 0;
  }
};

// ranges_utils.h:3-15: flat index of row i of the full batch grid inside a variable whose batch
// dimensions may be 1 (broadcast)
int64_t broadcast_index(int64_t i, int nbatchdims, const int64_t* full_shape, const int64_t* shape) {
  int64_t MN = shape[nbatchdims];
  int64_t res = i % MN, step = MN, full_step = MN;
  for (int b = nbatchdims; b > 0; b--) {
    if (shape[b - 1] != 1) res += ((i / full_step) % shape[b - 1]) * step;
    full_step *= full_shape[b - 1];
    step *= shape[b - 1];
  }
  return res;
}

// ---- module ------------------------------------------------------------------------------------

// set for the duration of keops_hip_launch_noalloc on the calling thread: nothing may be allocated or freed
thread_local bool g_noalloc = false;
// set while a host-pointer launch runs: its ranges are host memory, so they are validated on the host at every call
thread_local bool g_host_ranges = false;
// set while a use_half launch runs on the float32 copies of half-precision arguments
thread_local bool g_half_data = false;

struct DeviceBuffer {
  void* ptr = nullptr;
  size_t bytes = 0;
  bool frozen = false;    // a captured HIP graph holds pointers into this buffer: it is retired, not freed, when outgrown
  std::vector<void*> retired;
  bool borrowed = false;  // a view of memory owned elsewhere (the static scratch buffer): never freed, never grown
  int reserve(size_t n) {
    if (n <= bytes) return 0;
    if (borrowed)
      return fail(-1, "this call needs " + std::to_string(n) + " bytes of device workspace, more than the " + std::to_string(bytes) +
                      " bytes of the static scratch buffer of keops_hip_launch_noalloc");
    if (g_noalloc) return fail(-1, "keops_hip_launch_noalloc: this launch would allocate device memory");
    if (frozen && ptr) {
      // a HIP graph captured from this module holds pointers into the buffer: it stays alive (until the module is
      // destroyed) for the graph's replays, and this and later calls get a buffer of their own
      retired.push_back(ptr);
      ptr = nullptr;
      bytes = 0;
      frozen = false;
    }
    // (while a stream records into a HIP graph both calls are refused: a launch has to run once, with the same
    // shapes, before it is captured)
    if (ptr) {
      hipError_t e = hipFree(ptr);
      if (e != hipSuccess) return fail((int)e, std::string("hipFree of workspace failed: ") + hipGetErrorString(e));
    }
    ptr = nullptr;
    bytes = 0;
    hipError_t e = hipMalloc(&ptr, n);
    if (e != hipSuccess) {
      ptr = nullptr;
      return fail((int)e, std::string("hipMalloc of workspace failed: ") + hipGetErrorString(e));
    }
    bytes = n;
    return 0;
  }
  // gives up the current buffer without freeing it (a captured graph still uses it)
  void retire() {
    if (ptr && !borrowed) retired.push_back(ptr);
    ptr = nullptr;
    bytes = 0;
    frozen = false;
  }
  void release() {
    if (ptr && !borrowed) (void)hipFree(ptr);
    for (void* p : retired) (void)hipFree(p);
    retired.clear();
    ptr = nullptr;
    bytes = 0;
  }
};

struct Module {
  int device = 0, nargs = 0;
  hipModule_t mod = nullptr;
  std::map<std::string, std::string> meta;
  std::map<std::string, hipFunction_t> fns;
  int cu_count = 256;
  // geometry baked into the code object
  int block = 256, rows = 1, tile_j = 256, dimred = 1, dimout = 1, sizeof_t = 4, sizeof_acc = 4;
  int nrowvars = 0, ncolvars = 0, nparvars = 0;
  std::string scheme;
  DeviceBuffer partial;  // column-slab partial accumulators
  DeviceBuffer tables;   // lookup / offsets / synthesized ranges
  void* pinned = nullptr;  // staging for the tables
  size_t pinned_bytes = 0;
  hipEvent_t tables_copied = nullptr;
  bool tables_in_flight = false;
  std::vector<int64_t> tables_key;  // batch mode: shape signature of the cached tables
  int64_t cached_nblocks = 0;
  // block-sparse mode: signature (pointers, sizes, geometry) of the ranges the host path has read and validated, the
  // number of workgroups it found, and where the device path keeps its status word
  std::vector<int64_t> ranges_key;
  int64_t ranges_nblocks = 0;
  const unsigned* last_guard = nullptr;  // flag of the last launch's device-side choice between two kernel families
  int64_t ranges_work_total = 0;  // of the validated ranges: reduced rows swept, summed over the row ranges
  double ranges_pairs = 0.0;      // ... and their pairs
  // status words of the tables built on the device, in pinned host memory that the kernels write directly (no
  // read-back): [0] an index was clamped, [1] workgroups were dropped.  Sticky until the host has looked at them.
  unsigned* ranges_status = nullptr;      // host address
  unsigned* ranges_status_dev = nullptr;  // the same words as the device sees them
  DeviceBuffer staging;  // host-pointer launches (tagHostDevice = 0): device copies of the arguments and of out
  // a launch was recorded into a HIP graph: workspaces and tables keep their address and contents from then on
  bool captured = false;
  bool pinned_frozen = false;
  std::vector<void*> retired_pinned;
  // the module's workspaces are shared by all its launches: a launch on another stream waits for the previous one
  hipEvent_t last_done = nullptr;
  hipStream_t last_stream = nullptr;
  bool has_last = false;
  // timing
  bool timing = false;
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  double last_ms = -1.0;

  int meta_int(const char* k, int dflt) const {
    auto it = meta.find(k);
    return it == meta.end() ? dflt : std::atoi(it->second.c_str());
  }
  int fn(const char* name, hipFunction_t* f) {
    auto it = fns.find(name);
    if (it != fns.end()) { *f = it->second; return 0; }
    hipError_t e = hipModuleGetFunction(f, mod, name);
    if (e != hipSuccess) return fail((int)e, std::string("kernel '") + name + "' not found in module: " + hipGetErrorString(e));
    fns[name] = *f;
    return 0;
  }
};

// Device tables of a block-sparse or batched launch (Ranges.h:40-86, keops_nvrtc.cpp:152-248): one
// (range id, first row, end row) entry per workgroup of rows_per_block rows, the reduced-index ranges and,
// with batch dimensions, the first-row offsets of the variables for every workgroup -- in the order
// [row variables | reduced variables | parameters], or one entry per argument when by_arg is set.
struct RangeTables {
  const int64_t *lookup = nullptr, *slices_x = nullptr, *ranges_y = nullptr, *offsets = nullptr;
  int64_t nblocks = 0;
  // block-sparse mode: the caller's row ranges (device) and what the validating launch measured on the host
  const int64_t* rx = nullptr;
  int64_t nranges = 0;
  int64_t work_total = 0;   // reduced rows swept, summed over the row ranges
  double pairs = 0.0;       // pairs of the pattern
};

int ensure_pinned(Module& m, size_t bytes);

// must match struct KeopsRangeTables of kernels/keops_common.h
struct RangeHeader {
  const int64_t *lookup = nullptr, *slices_x = nullptr, *ranges_y = nullptr, *offsets = nullptr;
  int32_t nbatchdims = 0, nargs = 0;
};

// a block-sparse / batched launch of one of the matrix-core schemes
struct RangeLaunch {
  RangeTables tables;
  int nbatchdims = 0;
  bool user_ranges = false;
  RangeHeader header(int nargs) const {
    RangeHeader h;
    h.lookup = tables.lookup; h.slices_x = tables.slices_x; h.ranges_y = tables.ranges_y; h.offsets = tables.offsets;
    h.nbatchdims = nbatchdims; h.nargs = nargs;
    return h;
  }
};

// true while `stream` records into a HIP graph: launches that wait for the device cannot take part
bool stream_is_capturing(hipStream_t stream) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &st) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return st != hipStreamCaptureStatusNone;
}

// KEOPS_HIP_DEVICE_RANGES=0 keeps every block-sparse launch on the host path (read-back and validation per call)
bool device_ranges_enabled() {
  static const bool on = [] {
    const char* e = std::getenv("KEOPS_HIP_DEVICE_RANGES");
    return !(e && e[0] == '0');
  }();
  return on;
}

int prepare_range_tables(Module& m, const ShapeTable& S, int tagI, bool user_ranges, int64_t* const* ranges,
                         int64_t rows_total, int64_t cols_total, int64_t rows_per_block, bool by_arg, const std::vector<int>& rowvars,
                         const std::vector<int>& colvars, const std::vector<int>& vP, hipStream_t stream, RangeTables& rt) {
  const int64_t* rx_dev = nullptr;  // row ranges, device (user ranges only)
  std::vector<int64_t> rx_host;     // row ranges on the host
  int64_t nranges = 0;
  const int64_t *slices_dev = nullptr, *ry_dev = nullptr;
  const int nb = S.nbatchdims;
  const int nvars = by_arg ? m.nargs : m.nrowvars + m.ncolvars + m.nparvars;
  std::vector<int64_t> synth;  // batch mode: [slices (nbatches)] [ranges_y (2*nbatches)]
  std::vector<int64_t> range_work;  // block-sparse mode: reduced rows per row range

  std::vector<int64_t> ukey;  // signature of a block-sparse call
  if (user_ranges) {
    const int sel = tagI == 0 ? 0 : 3;
    nranges = ranges[6][sel];
    rx_dev = ranges[sel];
    slices_dev = ranges[sel + 1];
    ry_dev = ranges[sel + 2];
    const int64_t nred_u = ranges[6][sel + 2];
    ukey = {tagI, by_arg ? 1 : 0, rows_per_block, (int64_t)(intptr_t)rx_dev, (int64_t)(intptr_t)slices_dev,
            (int64_t)(intptr_t)ry_dev, nranges, ranges[6][sel + 1], nred_u, rows_total, cols_total};
    if (device_ranges_enabled() && !g_host_ranges && nb == 0 && nranges >= 0 && nred_u >= 0 && ukey == m.ranges_key && m.ranges_status) {
      // These ranges (same addresses, same sizes: the key is the identity of the buffers, not their contents) have
      // been read and validated by an earlier call: the table is now built on the device from their current
      // contents, with every index clamped to its axis.  No read-back, no synchronisation; the launch can be
      // recorded in a HIP graph.  What had to be clamped is reported through two sticky status words that the
      // kernels write into pinned host memory: keops_hip_ranges_status reads and clears them, and a launch that finds
      // them set by an earlier launch fails, so out-of-bounds ranges never go unnoticed.
      if (g_noalloc) return fail(-1, "keops_hip_launch_noalloc: block-sparse and batched launches build device tables");
      if (const unsigned pending = (m.ranges_status[0] ? 1u : 0u) | (m.ranges_status[1] ? 2u : 0u)) {
        m.ranges_status[0] = m.ranges_status[1] = 0u;
        return fail(-1, std::string("an earlier block-sparse launch of this module found its ranges invalid (") +
                        ((pending & 1u) ? "an index was out of bounds and has been clamped to its axis" : "") +
                        ((pending & 3u) == 3u ? "; " : "") +
                        ((pending & 2u) ? "the row ranges overlap so much that workgroups were dropped" : "") +
                        "): its result is not the reduction over the ranges as given");
      }
      const int64_t nblocks_max = std::max(nranges + rows_total / rows_per_block, m.ranges_nblocks);
      const size_t words = keops_static_range_build_words(nranges, nred_u, nblocks_max);
      const bool capturing = stream_is_capturing(stream);
      if (!capturing && m.tables.frozen && m.tables.ptr != nullptr) m.tables.retire();
      if (m.tables_in_flight) {
        HIP_TRY(hipEventSynchronize(m.tables_copied));
        m.tables_in_flight = false;
      }
      if (int rc = m.tables.reserve(words * sizeof(int64_t))) return rc;
      m.tables_key.clear();  // whatever batch tables the buffer held are gone
      long long* base = (long long*)m.tables.ptr;
      KeopsRangeBuild B;
      B.rx = (const long long*)rx_dev; B.sl = (const long long*)slices_dev; B.ry = (const long long*)ry_dev;
      B.nranges = nranges; B.nred = nred_u; B.rows_total = rows_total; B.cols_total = cols_total;
      B.rows_per_block = rows_per_block; B.nblocks_max = nblocks_max;
      B.lookup = base;
      B.sl_clean = B.lookup + 3 * nblocks_max;
      B.ry_clean = B.sl_clean + nranges;
      B.nb = B.ry_clean + 2 * nred_u;
      B.work = B.nb + nranges;
      B.order = B.work + nranges;
      B.offs = B.order + nranges;
      B.status = m.ranges_status_dev;
      if (int e = keops_static_build_ranges(&B, stream)) return fail(e, "building the range tables on the device failed");
      rt.nblocks = nblocks_max;
      rt.lookup = (const int64_t*)B.lookup;
      rt.offsets = nullptr;
      rt.slices_x = (const int64_t*)B.sl_clean;
      rt.ranges_y = (const int64_t*)B.ry_clean;
      rt.rx = rx_dev; rt.nranges = nranges; rt.work_total = m.ranges_work_total; rt.pairs = m.ranges_pairs;
      return 0;
    }
    rx_host.resize((size_t)2 * nranges);
    if (stream_is_capturing(stream))
      return fail(-1, "the first launch with a set of block-sparse ranges reads them back from the device to validate "
                      "them: it cannot be captured in a HIP graph (run the call once eagerly, then capture it)");
    // same synchronous read-back as the reference (keops_nvrtc.cpp:195-197)
    if (nranges) HIP_TRY(hipMemcpyAsync(rx_host.data(), rx_dev, sizeof(int64_t) * 2 * nranges, hipMemcpyDeviceToHost, stream));
    // the slices and reduced ranges too: workgroups are issued longest first (below)
    const int64_t nred = ranges[6][sel + 2];
    if (nranges < 0 || nred < 0) return fail(-1, "negative row count in the ranges");
    // the kernels read slices[range id] and sweep the reduced-index ranges it points to: one slice per row range
    if (ranges[6][sel + 1] != nranges)
      return fail(-1, "the ranges hold " + std::to_string(nranges) + " row ranges but " + std::to_string(ranges[6][sel + 1]) + " slices");
    std::vector<int64_t> sl_host((size_t)nranges), ry_host((size_t)2 * nred);
    if (nranges) HIP_TRY(hipMemcpyAsync(sl_host.data(), slices_dev, sizeof(int64_t) * nranges, hipMemcpyDeviceToHost, stream));
    if (nred) HIP_TRY(hipMemcpyAsync(ry_host.data(), ry_dev, sizeof(int64_t) * 2 * nred, hipMemcpyDeviceToHost, stream));
    HIP_TRY(hipStreamSynchronize(stream));
    // every reduced-index range must lie inside the reduced axis: the kernels sweep [start, end) unchecked
    for (int64_t k = 0; k < nred; k++)
      if (ry_host[2 * k] < 0 || ry_host[2 * k + 1] < ry_host[2 * k] || ry_host[2 * k + 1] > cols_total)
        return fail(-1, "reduced-index range " + std::to_string(k) + " = [" + std::to_string(ry_host[2 * k]) + ", " +
                        std::to_string(ry_host[2 * k + 1]) + ") is out of bounds (the reduced axis has " + std::to_string(cols_total) + " rows)");
    // reduced rows swept by the workgroups of every row range
    range_work.assign((size_t)nranges, 0);
    for (int64_t r = 0; r < nranges; r++) {
      const int64_t a = r == 0 ? 0 : sl_host[r - 1], b = sl_host[r];
      if (a < 0 || b < a || b > nred) return fail(-1, "slices of row range " + std::to_string(r) + " are out of bounds");
      for (int64_t k = a; k < b; k++) range_work[r] += ry_host[2 * k + 1] - ry_host[2 * k];
    }
  } else {
    // block-diagonal pattern, one range per batch (Ranges.h:40-86)
    nranges = S.nbatches;
    const int64_t R = tagI == 0 ? S.M : S.N, C = tagI == 0 ? S.N : S.M;
    rx_host.resize((size_t)2 * nranges);
    synth.resize((size_t)5 * nranges);  // [slices][ranges_y][row ranges]
    for (int64_t b = 0; b < nranges; b++) {
      rx_host[2 * b] = b * R;
      rx_host[2 * b + 1] = (b + 1) * R;
      synth[b] = b + 1;
      synth[nranges + 2 * b] = b * C;
      synth[nranges + 2 * b + 1] = (b + 1) * C;
      synth[3 * nranges + 2 * b] = b * R;
      synth[3 * nranges + 2 * b + 1] = (b + 1) * R;
    }
  }

  // lookup table: one entry per workgroup (keops_nvrtc.cpp:210-231)
  int64_t nblocks = 0;
  for (int64_t r = 0; r < nranges; r++) {
    const int64_t len = rx_host[2 * r + 1] - rx_host[2 * r];
    if (len < 0 || rx_host[2 * r] < 0 || rx_host[2 * r + 1] > rows_total)
      return fail(-1, "row range " + std::to_string(r) + " is out of bounds");
    nblocks += (len + rows_per_block - 1) / rows_per_block;
  }

  // batch mode tables only depend on the shapes: reuse them across calls
  std::vector<int64_t> key;
  bool reuse = false;
  if (!user_ranges) {
    key.push_back(tagI);
    key.push_back(by_arg ? 1 : 0);
    key.push_back(rows_per_block);
    key.insert(key.end(), S.shapes.begin(), S.shapes.end());
    reuse = key == m.tables_key && m.tables.ptr != nullptr;
  }
  const size_t n_lookup = (size_t)3 * nblocks, n_off = nb > 0 ? (size_t)nblocks * nvars : 0, n_syn = synth.size();
  const size_t total = n_lookup + n_off + n_syn;
  if (!reuse && total > 0) {
    if (g_noalloc) return fail(-1, "keops_hip_launch_noalloc: block-sparse and batched launches build device tables");
    if (m.tables.frozen && m.tables.ptr != nullptr) {
      // a HIP graph captured from this module reads the current tables (and may replay their upload from the pinned
      // staging buffer): both stay as they are for the graph, this call builds its tables in fresh buffers
      m.tables.retire();
      if (m.pinned) m.retired_pinned.push_back(m.pinned);
      m.pinned = nullptr;
      m.pinned_bytes = 0;
    }
    if (m.tables_in_flight) {
      HIP_TRY(hipEventSynchronize(m.tables_copied));
      m.tables_in_flight = false;
    }
    if (int rc = ensure_pinned(m, total * sizeof(int64_t))) return rc;
    int64_t* lk = (int64_t*)m.pinned;
    int64_t* off = lk + n_lookup;
    int64_t* syn = off + n_off;
    // Workgroups start in table order.  Block-sparse patterns give them very different amounts of work: the row
    // ranges with the longest sweeps go first, so that the last workgroups to start are the short ones and the
    // chip does not idle behind a few long stragglers.
    std::vector<int64_t> order((size_t)nranges);
    for (int64_t r = 0; r < nranges; r++) order[r] = r;
    if (!range_work.empty())
      std::stable_sort(order.begin(), order.end(), [&](int64_t a, int64_t b) { return range_work[a] > range_work[b]; });
    int64_t idx = 0;
    for (int64_t ro = 0; ro < nranges; ro++) {
      const int64_t r = order[ro];
      const int64_t s = rx_host[2 * r], len = rx_host[2 * r + 1] - s;
      for (int64_t j = 0; j < len; j += rows_per_block) {
        lk[3 * idx] = r;
        lk[3 * idx + 1] = s + j;
        lk[3 * idx + 2] = s + j + std::min(rows_per_block, len - j);
        idx++;
      }
    }
    if (nb > 0) {
      // per-block first-row offsets of every variable (keops_nvrtc.cpp:75-149, ranges_utils.h:27-91)
      const int W = nb + 3;
      const int64_t R = tagI == 0 ? S.M : S.N, C = tagI == 0 ? S.N : S.M;
      const int rpos = tagI == 0 ? nb : nb + 1, cpos = tagI == 0 ? nb + 1 : nb;
      std::vector<int64_t> shp(nb + 1);
      for (int64_t k = 0; k < nblocks; k++) {
        const int64_t rid = lk[3 * k];
        const int64_t patch = lk[3 * k + 1] - rid * R;
        int64_t* o = off + k * nvars;
        int c = 0;
        if (by_arg) std::fill(o, o + nvars, (int64_t)0);
        for (int v : rowvars) {
          const int64_t* r = S.row(v + 1);
          for (int b = 0; b < nb; b++) shp[b] = r[b];
          shp[nb] = r[rpos];
          o[by_arg ? v : c++] = patch + broadcast_index(rid * R, nb, S.shapes.data(), shp.data());
        }
        for (int v : colvars) {
          const int64_t* r = S.row(v + 1);
          for (int b = 0; b < nb; b++) shp[b] = r[b];
          shp[nb] = r[cpos];
          o[by_arg ? v : c++] = broadcast_index(rid * C, nb, S.shapes.data(), shp.data());
        }
        for (int v : vP) {
          const int64_t* r = S.row(v + 1);
          for (int b = 0; b < nb; b++) shp[b] = r[b];
          shp[nb] = 1;
          o[by_arg ? v : c++] = broadcast_index(rid, nb, S.shapes.data(), shp.data());
        }
        (void)W;
      }
    }
    if (n_syn) std::memcpy(syn, synth.data(), n_syn * sizeof(int64_t));
    // (block-sparse mode: room for the tables that later calls with these ranges build on the device)
    const size_t dev_words = (user_ranges && nb == 0)
        ? keops_static_range_build_words(nranges, ranges[6][(tagI == 0 ? 0 : 3) + 2], std::max(nranges + rows_total / rows_per_block, nblocks)) : 0;
    if (int rc = m.tables.reserve(std::max(total, dev_words) * sizeof(int64_t))) return rc;
    HIP_TRY(hipMemcpyAsync(m.tables.ptr, m.pinned, total * sizeof(int64_t), hipMemcpyHostToDevice, stream));
    if (!m.tables_copied) HIP_TRY(hipEventCreateWithFlags(&m.tables_copied, hipEventDisableTiming));
    HIP_TRY(hipEventRecord(m.tables_copied, stream));
    m.tables_in_flight = true;
    m.tables_key = key;
    m.cached_nblocks = nblocks;
  }
  if (user_ranges) {
    if (!m.ranges_status && !g_noalloc && !g_host_ranges) {
      HIP_TRY(hipHostMalloc((void**)&m.ranges_status, 64, hipHostMallocMapped));
      m.ranges_status[0] = m.ranges_status[1] = 0u;
      HIP_TRY(hipHostGetDevicePointer((void**)&m.ranges_status_dev, m.ranges_status, 0));
    }
    m.ranges_key = ukey;  // read and validated: later calls build the table on the device
    m.ranges_nblocks = nblocks;
    m.ranges_work_total = 0;
    m.ranges_pairs = 0.0;
    for (int64_t r = 0; r < nranges; r++) {
      m.ranges_work_total += range_work[r];
      m.ranges_pairs += (double)range_work[r] * (double)(rx_host[2 * r + 1] - rx_host[2 * r]);
    }
    rt.rx = rx_dev; rt.nranges = nranges; rt.work_total = m.ranges_work_total; rt.pairs = m.ranges_pairs;
  }
  const int64_t* tab = (const int64_t*)m.tables.ptr;
  rt.nblocks = nblocks;
  rt.lookup = tab;
  rt.offsets = nb > 0 ? tab + n_lookup : nullptr;
  if (user_ranges) {
    rt.slices_x = slices_dev;
    rt.ranges_y = ry_dev;
  } else {
    rt.slices_x = tab + n_lookup + n_off;
    rt.ranges_y = tab + n_lookup + n_off + nranges;
    // the batches as row ranges over the flattened arrays (kernels that give every range its own centre)
    const int64_t R = tagI == 0 ? S.M : S.N, C = tagI == 0 ? S.N : S.M;
    rt.rx = tab + n_lookup + n_off + 3 * nranges;
    rt.nranges = nranges;
    rt.work_total = nranges * C;
    rt.pairs = (double)nranges * (double)R * (double)C;
  }
  return 0;
}

// Kernel argument block: must match struct KeopsParams of kernels/keops_conv.h.
struct LaunchHeader {
  int64_t nx, ny;
  void* out;
  void* partial;
  int64_t slab_len;
  int32_t nslabs, nbatchdims;
  const int64_t* lookup;
  const int64_t* slices_x;
  const int64_t* ranges_y;
  const int64_t* offsets;
  const unsigned* guard;
};

int launch_raw3(Module& m, const char* kernel, unsigned gx, unsigned gy, unsigned gz, unsigned block, void* params,
                size_t size, hipStream_t stream) {
  hipFunction_t f;
  if (int rc = m.fn(kernel, &f)) return rc;
  void* extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, params, HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
  if (gx == 0 || gy == 0 || gz == 0) return 0;
  HIP_TRY(hipModuleLaunchKernel(f, gx, gy, gz, block, 1, 1, 0, stream, nullptr, extra));
  return 0;
}

int launch_raw(Module& m, const char* kernel, unsigned gx, unsigned gy, unsigned block, void* params, size_t size,
               hipStream_t stream) {
  return launch_raw3(m, kernel, gx, gy, 1, block, params, size, stream);
}

int launch(Module& m, const char* kernel, unsigned gx, unsigned gy, const LaunchHeader& h, void* const* args,
           hipStream_t stream) {
  std::vector<char> buf(sizeof(LaunchHeader) + sizeof(void*) * (size_t)std::max(1, m.nargs));
  std::memcpy(buf.data(), &h, sizeof(h));
  for (int k = 0; k < m.nargs; k++) std::memcpy(buf.data() + sizeof(h) + sizeof(void*) * k, &args[k], sizeof(void*));
  return launch_raw(m, kernel, gx, gy, (unsigned)m.block, buf.data(), buf.size(), stream);
}

int ensure_pinned(Module& m, size_t bytes) {
  if (bytes <= m.pinned_bytes) return 0;
  if (g_noalloc) return fail(-1, "keops_hip_launch_noalloc: this launch would allocate pinned host memory");
  if (m.pinned_frozen && m.pinned) {
    m.retired_pinned.push_back(m.pinned);  // a captured graph may replay copies from it
    m.pinned = nullptr;
    m.pinned_bytes = 0;
  }
  m.pinned_frozen = false;
  if (m.pinned) (void)hipHostFree(m.pinned);
  m.pinned = nullptr;
  m.pinned_bytes = 0;
  HIP_TRY(hipHostMalloc(&m.pinned, bytes, hipHostMallocDefault));
  m.pinned_bytes = bytes;
  return 0;
}

// ---- exponents of low-dimensional radial kernels on the matrix cores (kernels/keops_radial_mfma.h) ----

size_t align_up(size_t x, size_t a);

// must match struct RadParams of kernels/keops_radial_mfma.h (argument pointers follow)
struct RadHeader {
  int64_t nx, ny;
  void* xa;
  void* yb;
  void* bw;
  void* colsum;
  void* colpart;
  void* scal;
  void* hist[2];
  void* btot[2];
  void* bkt[2];
  void* perm[2];
  void* qn[2];
  void* gmax[2];
  void* out;
  void* partial;
  void* yo;
  void* xpart;
  void* segmax;
  int64_t slab_len, seg_len;
  int32_t nslabs, nseg, nparts;
};

// Launches the pre-pass (centre, counting sort of both clouds by their centred norms, slot vectors in sorted order,
// tile maxima), the decision kernel and the matrix-core sweep of a module built with radial=1, all asynchronous;
// *guard receives the device address of the flag that the general-purpose kernels, launched by the caller right
// after, test before doing anything.  Workspace: the first `reserved` bytes of m.partial stay free for the caller
// (slab partials of the general-purpose kernel).
int launch_radial(Module& m, int64_t nx, int64_t ny, void* out, void* const* args, hipStream_t stream, size_t reserved,
                  const unsigned** guard) {
  const int64_t D = m.meta_int("rad_d", 0), DV = m.meta_int("rad_dv", 0), NKB = m.meta_int("rad_nkb", 0);
  const int64_t RB = m.meta_int("rad_rb", 0), WAVES = m.meta_int("rad_waves", 0), TJ = m.meta_int("rad_tj", 128);
  const int64_t NBK = m.meta_int("rad_nbk", 128), CHUNK = m.meta_int("rad_sort_chunk", 1024);
  if (D <= 0 || DV <= 0 || NKB <= 0 || RB <= 0 || WAVES <= 0) return fail(-1, "corrupt radial module metadata");
  if (nx >= (int64_t)1 << 31 || ny >= ((int64_t)1 << 31) - TJ) return fail(-1, "radial scheme: more than 2^31 points");
  const int64_t ntiles = (ny + TJ - 1) / TJ, rows_per_wg = 32 * RB * WAVES, row_blocks = (nx + rows_per_wg - 1) / rows_per_wg;
  // slabs over the reduced axis: about 16 workgroups per compute unit, whole tiles per slab
  int64_t nslabs = std::max<int64_t>(1, (16 * (int64_t)m.cu_count + row_blocks - 1) / row_blocks);
  static const int64_t slab_cols = [] { const char* e = getenv("KEOPS_HIP_RADIAL_SLAB_COLS"); return e ? atoll(e) : 0; }();
  if (slab_cols > 0) nslabs = std::max<int64_t>(nslabs, (ny + slab_cols - 1) / slab_cols);
  nslabs = std::min<int64_t>(nslabs, std::max<int64_t>(1, ntiles / 8));
  int64_t slab_len = ((ny + nslabs - 1) / nslabs + TJ - 1) / TJ * TJ;
  nslabs = std::max<int64_t>(1, (ny + slab_len - 1) / slab_len);
  const int nparts = (int)std::max<int64_t>(1, std::min<int64_t>(256, ny / 1024));
  const int64_t ncols = ntiles * TJ;  // columns of the padded tile grid
  const int nblk_r = (int)((nx + CHUNK - 1) / CHUNK), nblk_c = (int)((ny + CHUNK - 1) / CHUNK);
  size_t off = align_up(reserved, 256);
  auto take = [&](size_t bytes) { size_t o = off; off = align_up(off + bytes, 256); return o; };
  const size_t o_scal = take(32), o_colsum = take((size_t)D * 4), o_colpart = take((size_t)nparts * D * 4);
  const size_t o_hist_r = take((size_t)NBK * nblk_r * 4), o_hist_c = take((size_t)NBK * nblk_c * 4);
  const size_t o_btot_r = take((size_t)NBK * 4), o_btot_c = take((size_t)NBK * 4);
  const size_t o_bkt_r = take((size_t)nx), o_bkt_c = take((size_t)ny);
  const size_t o_perm_r = take((size_t)nx * 4), o_perm_c = take((size_t)ncols * 4);
  const size_t o_qn_r = take((size_t)nx * 4), o_qn_c = take((size_t)ncols * 4);
  const int64_t groups_r = (nx + 32 * RB - 1) / (32 * RB);
  const size_t o_gmax_r = take((size_t)groups_r * 4), o_gmax_c = take((size_t)ntiles * 4);
  // weights of a column: RAD_DV floats, or 32 bfloat16 operand columns when the weighted sum runs on the matrix cores
  // (three terms of every weight: one block of 32 columns up to ten weights, rad_mm_nb blocks beyond)
  const size_t wbytes = m.meta_int("rad_mm", 0) != 0 ? 64 * (size_t)std::max<int64_t>(1, m.meta_int("rad_mm_nb", 1))
                                                      : (size_t)std::max<int64_t>(DV, m.meta_int("rad_ws", 0)) * 4;
  const size_t o_xa = take((size_t)nx * NKB * 32), o_yb = take((size_t)ncols * NKB * 32), o_bw = take((size_t)ncols * wbytes);
  const size_t o_part = take((size_t)nslabs * nx * DV * 4);
  // column segments of the kernel that computes the left-out tiles from exact differences: finer than the slabs (its
  // work sits in a corner of the pair matrix), at most 16 and at most 256 MiB of sums
  int64_t nseg = std::max<int64_t>(1, std::min<int64_t>(16, ((int64_t)256 << 20) / std::max<int64_t>(1, nx * DV * 4)));
  nseg = std::min<int64_t>(nseg, ntiles);
  const int64_t seg_len = ((ny + nseg - 1) / nseg + TJ - 1) / TJ * TJ;
  nseg = std::max<int64_t>(1, (ny + seg_len - 1) / seg_len);
  const size_t o_xpart = take((size_t)nseg * nx * DV * 4), o_segmax = take((size_t)nseg * 4);
  // what the exact kernel reads of a column, in sorted order: coordinates, centred coordinates (gradients), weights
  const int64_t XW = m.meta_int("rad_exact_xw", 8);
  const size_t o_yo = take((size_t)ncols * XW * 4);
  if (int rc = m.partial.reserve(off)) return rc;
  char* ws = (char*)m.partial.ptr;
  std::vector<char> buf(sizeof(RadHeader) + sizeof(void*) * (size_t)std::max(1, m.nargs) + 16);
  RadHeader h{};
  h.nx = nx; h.ny = ny; h.xa = ws + o_xa; h.yb = ws + o_yb; h.bw = ws + o_bw; h.colsum = ws + o_colsum; h.colpart = ws + o_colpart;
  h.scal = ws + o_scal;
  h.hist[0] = ws + o_hist_r; h.hist[1] = ws + o_hist_c; h.btot[0] = ws + o_btot_r; h.btot[1] = ws + o_btot_c; h.bkt[0] = ws + o_bkt_r; h.bkt[1] = ws + o_bkt_c;
  h.perm[0] = ws + o_perm_r; h.perm[1] = ws + o_perm_c; h.qn[0] = ws + o_qn_r; h.qn[1] = ws + o_qn_c;
  h.gmax[0] = ws + o_gmax_r; h.gmax[1] = ws + o_gmax_c;
  h.out = out; h.partial = ws + o_part; h.slab_len = slab_len; h.nslabs = (int32_t)nslabs; h.nparts = nparts;
  h.yo = ws + o_yo; h.xpart = ws + o_xpart; h.segmax = ws + o_segmax; h.seg_len = seg_len; h.nseg = (int32_t)nseg;
  std::memcpy(buf.data(), &h, sizeof(h));
  for (int k = 0; k < m.nargs; k++) std::memcpy(buf.data() + sizeof(h) + sizeof(void*) * k, &args[k], sizeof(void*));
  const size_t psize = sizeof(RadHeader) + sizeof(void*) * (size_t)std::max(1, m.nargs);
  auto with_which = [&](int w) { std::memcpy(buf.data() + psize, &w, 4); return psize + 4; };
  auto with_nblk = [&]() { std::memcpy(buf.data() + psize, &nblk_r, 4); std::memcpy(buf.data() + psize + 4, &nblk_c, 4); return psize + 8; };
  if (int rc = launch_raw(m, "keops_rad_colsum", (unsigned)nparts, 1, 256, buf.data(), psize, stream)) return rc;
  if (int rc = launch_raw(m, "keops_rad_colsum_final", 1, 1, 64, buf.data(), psize, stream)) return rc;
  if (int rc = launch_raw(m, "keops_rad_centre", (unsigned)D, 1, 256, buf.data(), psize, stream)) return rc;
  size_t sz = with_which(0);
  if (int rc = launch_raw(m, "keops_rad_bucket", (unsigned)nblk_r, 1, 256, buf.data(), sz, stream)) return rc;
  sz = with_which(1);
  if (int rc = launch_raw(m, "keops_rad_bucket", (unsigned)nblk_c, 1, 256, buf.data(), sz, stream)) return rc;
  sz = with_nblk();
  if (int rc = launch_raw(m, "keops_rad_scan", (unsigned)NBK, 2, 256, buf.data(), sz, stream)) return rc;
  if (int rc = launch_raw(m, "keops_rad_decide", 1, 1, (unsigned)NBK, buf.data(), psize, stream)) return rc;
  sz = with_which(0);
  if (int rc = launch_raw(m, "keops_rad_prep", (unsigned)nblk_r, 1, 256, buf.data(), sz, stream)) return rc;
  sz = with_which(1);
  if (int rc = launch_raw(m, "keops_rad_prep", (unsigned)((ncols + CHUNK - 1) / CHUNK), 1, 256, buf.data(), sz, stream)) return rc;
  if (int rc = launch_raw(m, "keops_rad_groupmax", (unsigned)((groups_r + ntiles + 3) / 4), 1, 256, buf.data(), psize, stream)) return rc;
  if (int rc = launch_raw(m, "keops_rad_segmax", (unsigned)nseg, 1, 64, buf.data(), psize, stream)) return rc;
  if (m.timing) HIP_TRY(hipEventRecord(m.ev0, stream));
  if (int rc = launch_raw(m, "keops_rad_main", (unsigned)row_blocks, (unsigned)nslabs, (unsigned)(64 * WAVES), buf.data(), psize, stream)) return rc;
  const int64_t xrows = m.meta_int("rad_exact_rows", 64);
  if (int rc = launch_raw(m, "keops_rad_exact", (unsigned)((nx + xrows - 1) / xrows), (unsigned)nseg, 256, buf.data(), psize, stream)) return rc;
  if (int rc = launch_raw(m, "keops_rad_reduce", (unsigned)((nx + 255) / 256), 1, 256, buf.data(), psize, stream)) return rc;
  *guard = (const unsigned*)(ws + o_scal) + 2;
  return 0;
}

// must match struct RadRParams of kernels/keops_radial_ranges.h (argument pointers follow)
struct RadRHeader {
  int64_t nx, ny, nranges, nblocks;
  const void* rx;
  RangeHeader rt;
  void *xa, *yb, *bw, *ctr, *vt, *rmax, *scal;
  int64_t vt_capacity;
  void *out, *partial;
};

// Block-sparse launches of a module built with radial=1 and rad_ranges=1: every row range gets its own centre and
// its own formatted copy of the columns it sweeps (kernels/keops_radial_ranges.h).  Worth it when the row ranges are
// long (the copy is one column per range and column, the work one pair per row and column) and the pattern holds
// enough pairs; otherwise *guard stays null and the general-purpose kernel runs alone.  All launches asynchronous.
int launch_radial_ranges(Module& m, int64_t nx, int64_t ny, void* out, void* const* args, hipStream_t stream, const RangeTables& rt,
                         const unsigned** guard) {
  *guard = nullptr;
  const int64_t D = m.meta_int("rad_d", 0), DV = m.meta_int("rad_dv", 0), NKB = m.meta_int("rad_nkb", 0);
  const int64_t RB = m.meta_int("rad_rb", 0), WAVES = m.meta_int("rad_waves", 0), TJ = m.meta_int("rad_tj", 128);
  if (D <= 0 || DV <= 0 || NKB <= 0 || RB <= 0 || WAVES <= 0) return fail(-1, "corrupt radial module metadata");
  const int64_t RPB = 32 * RB * WAVES;
  if (RPB != (int64_t)m.block * m.rows) return fail(-1, "corrupt radial module metadata: rows per workgroup");
  static const double min_pairs = [] {
    const char* e = std::getenv("KEOPS_HIP_RADIAL_RANGES_MIN_PAIRS");
    return e ? std::atof(e) : 268435456.0;  // 2^28, as for dense launches
  }();
  // rows per formatted column: at 128 the copy costs about a tenth of the sweep
  if (rt.nranges <= 0 || rt.pairs < min_pairs || rt.pairs < 128.0 * (double)rt.work_total || rt.nblocks < (int64_t)m.cu_count) return 0;
  const int64_t vt_capacity = rt.work_total / TJ + rt.nranges;  // every range pads less than one tile
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off = align_up(off + bytes, 256); return o; };
  const size_t o_scal = take(32), o_ctr = take((size_t)rt.nranges * D * 4), o_vt = take((size_t)rt.nranges * 16), o_rmax = take((size_t)rt.nranges * 8);
  const size_t o_xa = take((size_t)rt.nblocks * RPB * NKB * 32), o_yb = take((size_t)vt_capacity * TJ * NKB * 32);
  // weights of a formatted column: RAD_DV floats, or the operand columns of the second matrix product
  const size_t wbytes = m.meta_int("rad_mm", 0) != 0 ? 64 * (size_t)std::max<int64_t>(1, m.meta_int("rad_mm_nb", 1))
                                                      : (size_t)std::max<int64_t>(DV, m.meta_int("rad_ws", 0)) * 4;
  const size_t o_bw = take((size_t)vt_capacity * TJ * wbytes), o_part = take((size_t)rt.nblocks * RPB * DV * 4);
  if (off > ((size_t)4 << 30)) return 0;  // the formatted operands stay within 4 GiB
  if (int rc = m.partial.reserve(off)) return rc;
  char* ws = (char*)m.partial.ptr;
  std::vector<char> buf(sizeof(RadRHeader) + sizeof(void*) * (size_t)std::max(1, m.nargs));
  RadRHeader h{};
  h.nx = nx; h.ny = ny; h.nranges = rt.nranges; h.nblocks = rt.nblocks; h.rx = rt.rx;
  h.rt.lookup = rt.lookup; h.rt.slices_x = rt.slices_x; h.rt.ranges_y = rt.ranges_y; h.rt.offsets = nullptr;
  h.rt.nbatchdims = 0; h.rt.nargs = m.nargs;
  h.xa = ws + o_xa; h.yb = ws + o_yb; h.bw = ws + o_bw; h.ctr = ws + o_ctr; h.vt = ws + o_vt; h.rmax = ws + o_rmax; h.scal = ws + o_scal;
  h.vt_capacity = vt_capacity; h.out = out; h.partial = ws + o_part;
  std::memcpy(buf.data(), &h, sizeof(h));
  for (int k = 0; k < m.nargs; k++) std::memcpy(buf.data() + sizeof(h) + sizeof(void*) * k, &args[k], sizeof(void*));
  const size_t psize = buf.size();
  if (int rc = launch_raw(m, "keops_radr_centres", (unsigned)rt.nranges, 1, 256, buf.data(), psize, stream)) return rc;
  if (int rc = launch_raw(m, "keops_radr_scan", 1, 1, 1024, buf.data(), psize, stream)) return rc;
  if (int rc = launch_raw(m, "keops_radr_prep_rows", (unsigned)rt.nblocks, 1, (unsigned)RPB, buf.data(), psize, stream)) return rc;
  if (int rc = launch_raw(m, "keops_radr_prep_cols", (unsigned)rt.nranges, 8, 256, buf.data(), psize, stream)) return rc;
  if (int rc = launch_raw(m, "keops_radr_decide", 1, 1, 256, buf.data(), psize, stream)) return rc;
  if (int rc = launch_raw(m, "keops_radr_main", (unsigned)rt.nblocks, 1, (unsigned)(64 * WAVES), buf.data(), psize, stream)) return rc;
  if (int rc = launch_raw(m, "keops_radr_finish", (unsigned)rt.nblocks, 1, (unsigned)RPB, buf.data(), psize, stream)) return rc;
  *guard = (const unsigned*)(ws + o_scal) + 2;
  return 0;
}

// ---- K-nearest-neighbour scheme (kernels/keops_knn_mfma.h) ---------------------------------------

// must match struct KnnParams of kernels/keops_knn_mfma.h
struct KnnHeader {
  int64_t nq, nr;
  const void* xq;
  const void* yr;
  void* xh;
  void* yh;
  void* xkey;
  void* ykey;
  void* colsum;
  void* colpart;
  void* plist_d;
  void* plist_i;
  int64_t slab_len;
  int32_t nslabs, ref_step;
  void* out;
  void* thr;
  void* log;
  void* logcount;
  void* overflow;
  int64_t logcap;
  int32_t stage, fb;  // fb: device-side fallback of the two-phase schedule (see KnnParams)
  // filter on signed bytes (modules with knn_i8=1, two-phase launches; null otherwise)
  void *xq8, *yq8, *ykey_i, *xnorm_i, *xres, *thr_i, *scal;
  int64_t batch_rows, batch_cols;  // batches served as row ranges: indices relative to the batch
};

size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// number of reference slabs that gives about `per_cu` workgroups per compute unit; a slab holds at least
// min_tiles staged tiles (adaptive lists restart in every slab: longer slabs; fixed thresholds: short ones are fine)
int64_t pick_slabs(int64_t qblocks, int64_t nr, int64_t tile, int64_t cus, int64_t per_cu, int forced_min, int64_t min_tiles = 16) {
  int64_t n = std::max<int64_t>(1, (per_cu * cus) / std::max<int64_t>(1, qblocks));
  n = std::max<int64_t>(n, forced_min);
  n = std::min<int64_t>(n, std::max<int64_t>(1, nr / (min_tiles * tile)));
  return std::max<int64_t>(1, std::min<int64_t>(n, 1024));
}

// Workgroups that all take the same time run in rounds over the compute units: among the slab counts
// n0 .. nmax pick the one whose grid (blocks * n) fills its last round best (a larger count must win
// by 1.5 % to be preferred).
int64_t balance_slabs(int64_t blocks, int64_t n0, int64_t nmax, int64_t slots) {
  int64_t best = n0;
  double best_eff = 0.0;
  for (int64_t n = n0; n <= std::max(n0, nmax); n++) {
    const int64_t g = blocks * n, rounds = (g + slots - 1) / slots;
    const double eff = (double)g / (double)(rounds * slots);
    if (eff > best_eff + 0.015) { best_eff = eff; best = n; }
  }
  return best;
}

// smallest sample of the threshold estimate and smallest reference set handled in two phases (tuning knobs)
int64_t knn_min_sample() {
  static const int64_t v = [] { const char* e = getenv("KEOPS_HIP_KNN_MIN_SAMPLE"); return e ? std::max<int64_t>(64, atoll(e)) : 4096; }();
  return v;
}
int64_t knn_two_phase_min_refs() {
  static const int64_t v = [] { const char* e = getenv("KEOPS_HIP_KNN_TWO_PHASE_MIN"); return e ? std::max<int64_t>(1024, atoll(e)) : 16384; }();
  return v;
}

int launch_knn(Module& m, int64_t nq, int64_t nr, const void* xq, const void* yr, void* out, int tag1D2D,
               hipStream_t stream) {
  const int64_t D = m.meta_int("knn_d", 0), DP = m.meta_int("knn_dpad", 0), K = m.meta_int("knn_k", 0);
  const int64_t QB = m.meta_int("knn_qb", 256), TJ = m.tile_j, FTJ = m.meta_int("knn_ftj", m.tile_j);
  const int64_t FW = m.meta_int("knn_fwaves", 16), FQW = 32 * m.meta_int("knn_fqsets", 2);
  const int64_t FQB = FW * FQW;
  if (D <= 0 || DP <= 0 || K <= 0) return fail(-1, "corrupt knn module metadata");
  if (nr > 2147483647LL) return fail(-1, "too many reference rows for 32-bit indices");
  // sampling step of the threshold estimate: every 16th reference for large sets, a sample of >= ~4096 rows otherwise
  const int64_t SAMPLE = std::max<int64_t>(2, std::min<int64_t>(m.meta_int("knn_sample", 16), nr / knn_min_sample()));
  // (the two-phase schedule needs no read-back: when a candidate log overflows, the adaptive kernel, launched behind
  // it and idle otherwise, redoes the search, so the same sequence of launches also records into a HIP graph)
  const bool two_phase = nr >= knn_two_phase_min_refs() && nr / SAMPLE >= 8 * K && nq >= 1024;
  const int64_t nsample = two_phase ? (nr + SAMPLE - 1) / SAMPLE : 0;

  // adaptive pass: over the sample (two-phase) or over everything
  const int64_t a_nr = two_phase ? nsample : nr;
  const int64_t SQB = m.meta_int("knn_sqb", QB), SBLOCK = m.meta_int("knn_sblock", m.block);
  const int64_t a_qblocks = (nq + (two_phase ? SQB : QB) - 1) / (two_phase ? SQB : QB);
  static const int64_t main_per_cu = [] { const char* e = getenv("KEOPS_HIP_KNN_MAIN_PER_CU"); return e ? std::max<int64_t>(1, atoll(e)) : 2; }();
  static const int64_t main_min_tiles = [] { const char* e = getenv("KEOPS_HIP_KNN_MAIN_MIN_TILES"); return e ? std::max<int64_t>(1, atoll(e)) : 16; }();
  int64_t a_slabs = pick_slabs(a_qblocks, a_nr, TJ, m.cu_count, two_phase ? 2 : main_per_cu, tag1D2D == 1 && !two_phase ? 2 : 1,
                               two_phase ? 16 : main_min_tiles);
  int64_t a_len = ((a_nr + a_slabs - 1) / a_slabs + TJ - 1) / TJ * TJ;
  a_slabs = std::max<int64_t>(1, (a_nr + a_len - 1) / a_len);
  // filter pass
  const int64_t f_qblocks = (nq + FQB - 1) / FQB;
  int64_t f_slabs = pick_slabs(f_qblocks, nr, FTJ, m.cu_count, 2, 1, 4);
  // one filter workgroup fills a CU and all of them take the same time.  With at least 8 slabs the filter runs
  // in two stages (every 4th slab, then the others, with thresholds refined in between): both grids should
  // be close to whole rounds over the CUs
  {
    const int64_t cap = std::max<int64_t>(1, nr / (4 * FTJ));
    int64_t best = f_slabs;
    double best_eff = 0.0;
    for (int64_t n = f_slabs; n <= std::max(f_slabs, std::min<int64_t>(std::max<int64_t>(4 * f_slabs, 24), cap)); n++) {
      auto eff = [&](int64_t blocks) {
        const int64_t rounds = (blocks + m.cu_count - 1) / m.cu_count;
        return (double)blocks / (double)(rounds * m.cu_count);
      };
      const int64_t na = n >= 8 ? (n + 3) / 4 : n;
      const double e = n >= 8 ? (eff(f_qblocks * na) + 3.0 * eff(f_qblocks * (n - na))) / 4.0 : eff(f_qblocks * n);
      if (e > best_eff + 0.015) { best_eff = e; best = n; }
    }
    f_slabs = best;
  }
  int64_t f_len = ((nr + f_slabs - 1) / f_slabs + FTJ - 1) / FTJ * FTJ;
  f_slabs = std::max<int64_t>(1, (nr + f_len - 1) / f_len);
  const bool staged = two_phase && f_slabs >= 8;
  const int64_t fa_slabs = staged ? (f_slabs + 3) / 4 : f_slabs, fb_slabs = f_slabs - fa_slabs;
  const int64_t nlogs = f_qblocks * f_slabs * FW;
  // expected survivors per query: SAMPLE * K (the sample's K-th neighbour is about the (SAMPLE*K)-th overall)
  const int64_t logcap = two_phase ? align_up((size_t)(5 * FQW * SAMPLE * K / f_slabs + 512), 64) : 0;
  const int64_t list_slabs = std::max<int64_t>(a_slabs, two_phase ? f_slabs : 1);

  // workspace layout
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off = align_up(off + bytes, 256); return o; };
  const int nparts = (int)std::max<int64_t>(1, std::min<int64_t>(512, nr / 64));
  // (two more rows of colpart: medians and flag of keops_knn_centre)
  const size_t o_colsum = take((size_t)DP * 4), o_colpart = take((size_t)(nparts + 2) * DP * 4);
  const int64_t RW = DP * (m.meta_int("knn_split", 0) ? 2 : 1);  // bf16 elements per stored row ([hi] or [hi | lo])
  const size_t o_xh = take((size_t)nq * RW * 2), o_yh = take((size_t)nr * RW * 2);
  const size_t o_xkey = take((size_t)nq * 4), o_ykey = take((size_t)nr * 4);
  const size_t o_pd = take((size_t)list_slabs * nq * K * 4), o_pi = take((size_t)list_slabs * nq * K * 4);
  const size_t o_yhs = take((size_t)nsample * RW * 2), o_ykeys = take((size_t)nsample * 4);
  const size_t o_thr = take((size_t)nq * 4), o_flag = take(256);
  const size_t o_logcount = take((size_t)(two_phase ? nlogs : 0) * 4), o_log = take((size_t)(two_phase ? nlogs : 0) * logcap * 8);
  // the filter also runs on signed bytes (twice the matrix rate, half the staged bytes) when the device finds its
  // slack small against the search radii
  const bool i8 = two_phase && m.meta_int("knn_i8", 0) != 0;
  const int64_t DP8 = (D + 31) / 32 * 32;
  const size_t o_xq8 = take(i8 ? (size_t)nq * DP8 : 0), o_yq8 = take(i8 ? (size_t)nr * DP8 : 0);
  const size_t o_ykeyi = take(i8 ? (size_t)nr * 4 : 0), o_xnormi = take(i8 ? (size_t)nq * 4 : 0), o_thri = take(i8 ? (size_t)nq * 4 : 0);
  const size_t o_xres = take(i8 ? (size_t)nq * 4 : 0);
  const size_t o_scal = take(64);
  if (int rc = m.partial.reserve(off)) return rc;
  char* ws = (char*)m.partial.ptr;
  struct Packed { KnnHeader h; int64_t extra[4]; } p{};
  KnnHeader& h = p.h;
  h.nq = nq; h.nr = nr; h.xq = xq; h.yr = yr;
  h.xh = ws + o_xh; h.yh = ws + o_yh; h.xkey = ws + o_xkey; h.ykey = ws + o_ykey; h.colsum = ws + o_colsum; h.colpart = ws + o_colpart;
  h.plist_d = ws + o_pd; h.plist_i = ws + o_pi; h.out = out; h.ref_step = 1;
  h.thr = ws + o_thr; h.log = ws + o_log; h.logcount = ws + o_logcount; h.overflow = ws + o_flag; h.logcap = logcap;
  if (i8) {
    h.xq8 = ws + o_xq8; h.yq8 = ws + o_yq8; h.ykey_i = ws + o_ykeyi; h.xnorm_i = ws + o_xnormi; h.xres = ws + o_xres;
    h.thr_i = ws + o_thri; h.scal = ws + o_scal;
  }
  m.last_guard = i8 ? (const unsigned*)(ws + o_scal) + 3 : nullptr;
  const size_t HS = sizeof(KnnHeader);
  auto run = [&](const char* k, unsigned gx, unsigned gy, unsigned block, size_t size) {
    return launch_raw(m, k, gx, gy, block, &p, size, stream);
  };
  auto with_int = [&](int v) { std::memcpy(p.extra, &v, 4); return HS + 4; };

  // pre-pass: centring, bf16 copies, keys
  if (int rc = run("keops_knn_colsum", (unsigned)nparts, 1, 256, HS)) return rc;
  if (int rc = run("keops_knn_colsum_final", 1, 1, 256, with_int(nparts))) return rc;
  if (int rc = run("keops_knn_centre", (unsigned)D, 1, 256, with_int(nparts))) return rc;
  if (int rc = run("keops_knn_centre_apply", 1, 1, 256, with_int(nparts))) return rc;
  const int64_t lpr = DP / 4 <= 4 ? 4 : (DP / 4 <= 8 ? 8 : (DP / 4 <= 16 ? 16 : (DP / 4 <= 32 ? 32 : 64)));
  if (int rc = run("keops_knn_prep", (unsigned)((nq * lpr + 255) / 256), 1, 256, with_int(0))) return rc;
  if (int rc = run("keops_knn_prep", (unsigned)((nr * lpr + 255) / 256), 1, 256, with_int(1))) return rc;
  if (i8) {
    // (after both bf16 passes: they find the largest centred component, which sets the quantisation step)
    const int64_t lpr8 = DP8 / 4 <= 8 ? 8 : (DP8 / 4 <= 16 ? 16 : (DP8 / 4 <= 32 ? 32 : 64));
    if (int rc = run("keops_knn_quant", (unsigned)((nq * lpr8 + 255) / 256), 1, 256, with_int(0))) return rc;
    if (int rc = run("keops_knn_quant", (unsigned)((nr * lpr8 + 255) / 256), 1, 256, with_int(1))) return rc;
  }
  if (m.timing) HIP_TRY(hipEventRecord(m.ev0, stream));

  auto adaptive = [&](const char* kernel, int64_t refs, void* yh, void* ykey, int step, int64_t slabs, int64_t len) -> int {
    h.nr = refs; h.yh = yh; h.ykey = ykey; h.ref_step = step; h.nslabs = (int32_t)slabs; h.slab_len = len;
    const bool sampling = step > 1;
    const int64_t qb = sampling ? SQB : QB;
    return run(kernel, (unsigned)((nq + qb - 1) / qb), (unsigned)slabs, (unsigned)(sampling ? SBLOCK : m.block), HS);
  };
  if (two_phase) {
    // (a) thresholds from every SAMPLE-th reference
    void* gargs[3] = {ws + o_yhs, ws + o_ykeys, nullptr};
    std::memcpy(&p.extra[0], &gargs[0], 8);
    std::memcpy(&p.extra[1], &gargs[1], 8);
    p.extra[2] = nsample;
    p.extra[3] = SAMPLE;  // read as a 32-bit integer (little endian)
    const int64_t chunks = nsample * (RW / 8);
    if (int rc = run("keops_knn_gather_sample", (unsigned)((chunks + 255) / 256), 1, 256, HS + 32)) return rc;
    if (int rc = adaptive("keops_knn_sample", nsample, ws + o_yhs, ws + o_ykeys, (int)SAMPLE, a_slabs, a_len)) return rc;
    auto with_2int = [&](int a, int b) { int v[2] = {a, b}; std::memcpy(p.extra, v, 8); return HS + 8; };
    if (int rc = run("keops_knn_thresholds", (unsigned)((nq + 255) / 256), 1, 256, with_2int(0, 0))) return rc;
    // (b) fixed-threshold filter, survivors logged per wavefront; (c) exact replay of the logs.
    // Staged: every 4th slab first, thresholds refined from its replay, then the other slabs.
    h.nr = nr; h.yh = ws + o_yh; h.ykey = ws + o_ykey; h.ref_step = 1; h.nslabs = (int32_t)f_slabs; h.slab_len = f_len;
    h.stage = staged ? 1 : 0;
    // (one of the two filters returns at once: the choice was made on the device by keops_knn_thresholds)
    if (i8)
      if (int rc = run("keops_knn_filter_i8", (unsigned)f_qblocks, (unsigned)fa_slabs, (unsigned)(64 * FW), HS)) return rc;
    if (int rc = run("keops_knn_filter", (unsigned)f_qblocks, (unsigned)fa_slabs, (unsigned)(64 * FW), HS)) return rc;
    if (int rc = run("keops_knn_rerank", (unsigned)(f_qblocks * fa_slabs * FW), 1, 64, with_int((int)f_qblocks))) return rc;
    if (staged) {
      if (int rc = run("keops_knn_thresholds", (unsigned)((nq + 255) / 256), 1, 256, with_2int(1, (int)fa_slabs))) return rc;
      h.stage = 2;
      if (i8)
        if (int rc = run("keops_knn_filter_i8", (unsigned)f_qblocks, (unsigned)fb_slabs, (unsigned)(64 * FW), HS)) return rc;
      if (int rc = run("keops_knn_filter", (unsigned)f_qblocks, (unsigned)fb_slabs, (unsigned)(64 * FW), HS)) return rc;
      if (int rc = run("keops_knn_rerank", (unsigned)(f_qblocks * fb_slabs * FW), 1, 64, with_int((int)f_qblocks))) return rc;
      h.stage = 0;
    }
  }
  {
    // adaptive schedule: the whole search when the call is too small for two phases, else the fallback that only
    // runs when a log overflowed (pathological ties; decided on the device: the flag is never read back)
    int64_t slabs = pick_slabs((nq + QB - 1) / QB, nr, TJ, m.cu_count, main_per_cu, tag1D2D == 1 ? 2 : 1, main_min_tiles);
    slabs = std::min<int64_t>(slabs, list_slabs);
    int64_t len = ((nr + slabs - 1) / slabs + TJ - 1) / TJ * TJ;
    slabs = std::max<int64_t>(1, (nr + len - 1) / len);
    h.fb = two_phase ? 1 : 0;
    if (int rc = adaptive("keops_knn_main", nr, ws + o_yh, ws + o_ykey, 1, slabs, len)) return rc;
    if (two_phase) {
      // the merge reads the lists of whichever pass produced them
      h.nslabs = (int32_t)f_slabs;
      h.fb = (int32_t)slabs;
    }
  }
  if (m.timing) HIP_TRY(hipEventRecord(m.ev1, stream));
  if (int rc = run("keops_knn_merge", (unsigned)((nq + 255) / 256), 1, 256, HS)) return rc;
  return 0;
}

// Block-sparse launch of a K-nearest-neighbour module built for ranges (KNN_RANGES): pre-pass, neutral lists, the
// adaptive kernel with one workgroup per patch of a row range, merge (which writes the output layout).
int launch_knn_ranges(Module& m, int64_t nq, int64_t nr, const void* xq, const void* yr, void* out, hipStream_t stream,
                      const RangeLaunch& rg, int64_t batch_rows = 0, int64_t batch_cols = 0) {
  const int64_t D = m.meta_int("knn_d", 0), DP = m.meta_int("knn_dpad", 0), K = m.meta_int("knn_k", 0);
  if (D <= 0 || DP <= 0 || K <= 0) return fail(-1, "corrupt knn module metadata");
  if (nr > 2147483647LL) return fail(-1, "too many reference rows for 32-bit indices");
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off = align_up(off + bytes, 256); return o; };
  const int nparts = (int)std::max<int64_t>(1, std::min<int64_t>(512, nr / 64));
  // (two more rows of colpart: medians and flag of keops_knn_centre)
  const size_t o_colsum = take((size_t)DP * 4), o_colpart = take((size_t)(nparts + 2) * DP * 4);
  const int64_t RW = DP * (m.meta_int("knn_split", 0) ? 2 : 1);
  const size_t o_xh = take((size_t)nq * RW * 2), o_yh = take((size_t)nr * RW * 2);
  const size_t o_xkey = take((size_t)nq * 4), o_ykey = take((size_t)nr * 4);
  const size_t o_pd = take((size_t)nq * K * 4), o_pi = take((size_t)nq * K * 4);
  if (int rc = m.partial.reserve(off)) return rc;
  char* ws = (char*)m.partial.ptr;
  struct Packed { KnnHeader h; RangeHeader rt; int64_t extra[2]; } p{};
  static_assert(sizeof(KnnHeader) % 8 == 0, "the range tables follow the header without padding");
  KnnHeader& h = p.h;
  h.nq = nq; h.nr = nr; h.xq = xq; h.yr = yr;
  h.xh = ws + o_xh; h.yh = ws + o_yh; h.xkey = ws + o_xkey; h.ykey = ws + o_ykey; h.colsum = ws + o_colsum; h.colpart = ws + o_colpart;
  h.plist_d = ws + o_pd; h.plist_i = ws + o_pi; h.out = out; h.ref_step = 1; h.nslabs = 1; h.slab_len = nr;
  h.batch_rows = batch_rows; h.batch_cols = batch_cols;
  p.rt = rg.header(m.nargs);
  const size_t HS = sizeof(KnnHeader) + sizeof(RangeHeader);
  auto run = [&](const char* k, unsigned gx, unsigned block, size_t size) { return launch_raw(m, k, gx, 1, block, &p, size, stream); };
  auto with_int = [&](int v) { std::memcpy(p.extra, &v, 4); return HS + 4; };
  if (int rc = run("keops_knn_colsum", (unsigned)nparts, 256, HS)) return rc;
  if (int rc = run("keops_knn_colsum_final", 1, 256, with_int(nparts))) return rc;
  if (int rc = run("keops_knn_centre", (unsigned)D, 256, with_int(nparts))) return rc;
  if (int rc = run("keops_knn_centre_apply", 1, 256, with_int(nparts))) return rc;
  const int64_t lpr = DP / 4 <= 4 ? 4 : (DP / 4 <= 8 ? 8 : (DP / 4 <= 16 ? 16 : (DP / 4 <= 32 ? 32 : 64)));
  if (int rc = run("keops_knn_prep", (unsigned)((nq * lpr + 255) / 256), 256, with_int(0))) return rc;
  if (int rc = run("keops_knn_prep", (unsigned)((nr * lpr + 255) / 256), 256, with_int(1))) return rc;
  if (int rc = run("keops_knn_fill_lists", (unsigned)((nq * K + 255) / 256), 256, HS)) return rc;
  if (m.timing) HIP_TRY(hipEventRecord(m.ev0, stream));
  if (int rc = run("keops_knn_main", (unsigned)rg.tables.nblocks, (unsigned)m.block, HS)) return rc;
  if (m.timing) HIP_TRY(hipEventRecord(m.ev1, stream));
  if (int rc = run("keops_knn_merge", (unsigned)((nq + 255) / 256), 256, HS)) return rc;
  return 0;
}

// ---- matrix-core chunked scheme (kernels/keops_chunk_mfma.h) ---------------------------------------

// must match struct ChkParams of kernels/keops_chunk_mfma.h (argument pointers follow)
struct ChkHeader {
  int64_t nx, ny;
  void* xs;
  void* ys;
  void* xn;
  void* yn;
  void* colsum;
  void* colpart;
  void* out;
  void* partial;
  int64_t slab_len;
  int32_t nslabs;
  int32_t pad_;
  int64_t nxs, nys;
  void* vsplit;
  void* scal;
  RangeHeader rt;
};

// rg: block-sparse / batched launch (module built with ranges=1), else null; nxs, nys: rows of the chunked arguments
int launch_chunk(Module& m, int64_t nx, int64_t ny, void* out, void* const* args, int tag1D2D, hipStream_t stream,
                 const RangeLaunch* rg, int64_t nxs, int64_t nys) {
  const int64_t D = m.meta_int("chk_d", 0), DP = m.meta_int("chk_dpad", 0), QB = m.meta_int("chk_qb", 128);
  const int mode = m.meta_int("chk_mode", 0);
  if (D <= 0 || DP <= 0) return fail(-1, "corrupt chunk module metadata");
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off = align_up(off + bytes, 256); return o; };
  const int nparts = (int)std::max<int64_t>(1, std::min<int64_t>(128, nys / 64));
  // (one more row of colpart: the medians of keops_chk_centre)
  const size_t o_colsum = take((size_t)DP * 4), o_colpart = take((size_t)(nparts + 1) * DP * 4);
  // one half-precision term per component when the data are half-precision numbers (no lo parts, no centring)
  const bool single = m.meta_int("chk_single", 0) != 0;
  // one half-precision term per component is only exact for data that IS half precision
  if (single != g_half_data)
    return fail(-1, single ? "this module was compiled for half-precision data (use_half = 1 in get_keops_dll): launch it with "
                             "use_half = 1; float32 operands would be truncated to 11 bits"
                           : "this module was compiled for float32 data: a use_half launch needs the module that get_keops_dll "
                             "returns for use_half = 1");
  const size_t o_xs = take((size_t)nxs * DP * (single ? 2 : 4)), o_ys = take((size_t)nys * DP * (single ? 2 : 4));
  const size_t o_xn = take((size_t)nxs * 4), o_yn = take((size_t)nys * 4), o_scal = take(16 + 2 * 256 * 4);
  // final-product variant: slabs over the reduced axis fill the chip and round the grid to whole
  // rounds of workgroups (one 8-wavefront workgroup per CU, all taking the same time)
  const bool softmax = m.meta_int("chk_softmax", 0) != 0;
  const bool final = m.meta_int("chk_final", 0) != 0 || softmax;
  const int64_t row_blocks = rg ? rg->tables.nblocks : (nx + QB - 1) / QB, TJ = m.tile_j;
  int64_t nslabs = 1, slab_len = std::max<int64_t>(TJ, (ny + TJ - 1) / TJ * TJ);
  if (final && !rg) {
    const int64_t cap = std::max<int64_t>(1, ny / (8 * TJ));
    const int64_t target = 2 * (int64_t)m.cu_count;
    if (tag1D2D == 1 || row_blocks < target) {
      nslabs = std::min<int64_t>(cap, (target + row_blocks - 1) / row_blocks);
      if (tag1D2D == 1) nslabs = std::max<int64_t>(nslabs, std::min<int64_t>(cap, 2));
      nslabs = std::max<int64_t>(1, std::min<int64_t>(nslabs, 65535));
    }
    nslabs = balance_slabs(row_blocks, nslabs, std::min<int64_t>(std::max<int64_t>(nslabs, 8), cap), m.cu_count);
    slab_len = std::max<int64_t>(TJ, ((ny + nslabs - 1) / nslabs + TJ - 1) / TJ * TJ);
    nslabs = std::max<int64_t>(1, (ny + slab_len - 1) / slab_len);
  }
  const size_t o_part = take(final && nslabs > 1 ? (size_t)nslabs * nx * m.dimred * 4 : 0);
  // weighted sums with three-term bfloat16 operands (dense launches): pre-split copy of v, tile by tile
  const bool split3 = final && !rg && m.meta_int("chk_split3", 0) != 0;
  const int64_t vcols = m.meta_int("chk_vcols", 0), ntiles = (ny + TJ - 1) / TJ;
  const size_t o_vsplit = take(split3 ? (size_t)ntiles * 3 * vcols * 40 * 2 : 0);
  // K nearest neighbours in high dimension: the sweep keeps knn_inner > K approximate candidates per row in the
  // workspace, a second kernel re-ranks them exactly into `out` and counts the rows it cannot certify
  const int64_t knn_inner = m.meta_int("chk_knn_inner", 0);
  if (knn_inner > 0 && (rg || final)) return fail(-1, "corrupt chunk module metadata");
  if (knn_inner > 0) {
    // column slabs fill the chip (one workgroup per CU at these operand sizes); the re-rank gives one lane to every
    // candidate of a row: at most 64 / knn_inner slabs
    const int64_t cap = std::max<int64_t>(1, std::min<int64_t>(64 / knn_inner, ny / (16 * TJ)));
    const int64_t n0 = std::max<int64_t>(1, std::min<int64_t>(cap, (m.cu_count + row_blocks - 1) / row_blocks));
    nslabs = balance_slabs(row_blocks, n0, cap, m.cu_count);
    slab_len = std::max<int64_t>(TJ, ((ny + nslabs - 1) / nslabs + TJ - 1) / TJ * TJ);
    nslabs = std::max<int64_t>(1, (ny + slab_len - 1) / slab_len);
  }
  const size_t o_lists = take(knn_inner > 0 ? (size_t)nslabs * nx * 2 * knn_inner * 4 : 0), o_flag = take(knn_inner > 0 ? 256 : 0);
  if (knn_inner > 0 && stream_is_capturing(stream))
    return fail(-1, "this K-nearest-neighbour launch reads a flag back from the device: it cannot be captured in a HIP graph");
  if (int rc = m.partial.reserve(off)) return rc;
  char* ws = (char*)m.partial.ptr;
  std::vector<char> buf(sizeof(ChkHeader) + sizeof(void*) * (size_t)std::max(1, m.nargs) + 32);
  ChkHeader h{};
  h.nx = nx; h.ny = ny; h.xs = ws + o_xs; h.ys = ws + o_ys; h.xn = ws + o_xn; h.yn = ws + o_yn; h.colsum = ws + o_colsum;
  h.colpart = ws + o_colpart; h.out = out; h.partial = ws + o_part; h.slab_len = slab_len; h.nslabs = (int32_t)nslabs;
  h.nxs = nxs; h.nys = nys; h.scal = ws + o_scal;
  if (split3) h.vsplit = ws + o_vsplit;
  if (rg) h.rt = rg->header(m.nargs);
  if (knn_inner > 0) h.out = ws + o_lists;
  std::memcpy(buf.data(), &h, sizeof(h));
  for (int k = 0; k < m.nargs; k++) std::memcpy(buf.data() + sizeof(h) + sizeof(void*) * k, &args[k], sizeof(void*));
  const size_t psize = sizeof(ChkHeader) + sizeof(void*) * (size_t)std::max(1, m.nargs);
  int32_t which = 0;
  auto with_which = [&](int w) { which = w; std::memcpy(buf.data() + psize, &which, 4); return psize + 4; };
  if (mode == 0 && !single) {
    if (int rc = launch_raw(m, "keops_chk_colsum", (unsigned)nparts, 1, 256, buf.data(), psize, stream)) return rc;
    const size_t szp = with_which(nparts);
    const int64_t cw = D > 128 ? 256 : (D > 64 ? 128 : (D > 32 ? 64 : 32));  // CHK_CW: columns per workgroup
    if (int rc = launch_raw(m, "keops_chk_colsum_final", (unsigned)((DP + cw - 1) / cw), 1, 256, buf.data(), szp, stream)) return rc;
  }
  // power-of-two scales of the half-precision operands: largest |component| of both arguments
  if (int e = keops_static_fill_zero(ws + o_scal, 16 + 2 * 256 * 4, stream)) return fail(e, std::string("zero fill failed: ") + hipGetErrorString((hipError_t)e));
  {
    const int64_t elems = std::max(nxs, nys) * D;
    const unsigned gb = (unsigned)std::max<int64_t>(1, std::min<int64_t>(2048, (elems + 256 * 8 - 1) / (256 * 8)));
    if (int rc = launch_raw(m, "keops_chk_absmax", gb, 1, 256, buf.data(), psize, stream)) return rc;
  }
  // squared distances: the centre is the median of a sample when the mean is far from it (a few rows far away)
  if (mode == 0 && !single && m.meta_int("chk_robust", 0) != 0) {
    const size_t szc = with_which(nparts);
    if (int rc = launch_raw(m, "keops_chk_centre", (unsigned)D, 1, 256, buf.data(), szc, stream)) return rc;
    if (int rc = launch_raw(m, "keops_chk_centre_apply", 1, 1, 256, buf.data(), szc, stream)) return rc;
  }
  // squared distances: when a few rows hold components far beyond the others', the scale follows the bulk of the rows
  // and those rows are computed pair by pair from the float32 data (kernels/keops_chunk_mfma.h, keops_chk_robust)
  if (!single && m.meta_int("chk_robust", 0) != 0) {
    for (int w = 0; w < 2; w++) {
      const int64_t rows = w ? nys : nxs;
      const unsigned gb = (unsigned)std::max<int64_t>(1, std::min<int64_t>(1024, (rows + 31) / 32));
      const size_t szh = with_which(w);
      if (int rc = launch_raw(m, "keops_chk_rowhist", gb, 1, 256, buf.data(), szh, stream)) return rc;
    }
    if (int rc = launch_raw(m, "keops_chk_robust", 1, 1, 64, buf.data(), psize, stream)) return rc;
  }
  const int64_t lpr = DP / 4 <= 4 ? 4 : (DP / 4 <= 8 ? 8 : (DP / 4 <= 16 ? 16 : (DP / 4 <= 32 ? 32 : 64)));
  size_t sz = with_which(0);
  if (int rc = launch_raw(m, "keops_chk_prep", (unsigned)((nxs * lpr + 255) / 256), 1, 256, buf.data(), sz, stream)) return rc;
  sz = with_which(1);
  if (int rc = launch_raw(m, "keops_chk_prep", (unsigned)((nys * lpr + 255) / 256), 1, 256, buf.data(), sz, stream)) return rc;
  if (split3)
    if (int rc = launch_raw(m, "keops_chk_split", (unsigned)((ntiles * vcols * TJ + 255) / 256), 1, 256, buf.data(), psize, stream)) return rc;
  if (rg && rg->user_ranges)
    if (int rc = launch_raw(m, "keops_chk_fill_neutral", (unsigned)((nx + 255) / 256), 1, 256, buf.data(), psize, stream)) return rc;
  if (m.timing) HIP_TRY(hipEventRecord(m.ev0, stream));
  if (final) {
    if (int rc = launch_raw(m, softmax ? "keops_chk_softmax" : "keops_chk_final", (unsigned)row_blocks, (unsigned)nslabs, (unsigned)m.block, buf.data(), psize, stream)) return rc;
  } else {
    if (int rc = launch_raw(m, "keops_chk_main", (unsigned)row_blocks, (unsigned)(knn_inner > 0 ? nslabs : 1), (unsigned)m.block, buf.data(), psize, stream)) return rc;
  }
  if (m.timing) HIP_TRY(hipEventRecord(m.ev1, stream));
  if (final && nslabs > 1) {
    const int64_t gb = (nx * m.dimred + 255) / 256;
    if (int rc = launch_raw(m, softmax ? "keops_chk_softmax_reduce" : "keops_chk_reduce", (unsigned)gb, 1, 256, buf.data(), psize, stream)) return rc;
  }
  if (knn_inner > 0) {
    void* extra[3] = {ws + o_lists, out, ws + o_flag};  // struct ChkKnnExtra of kernels/keops_chunk_mfma.h
    std::memcpy(buf.data() + psize, extra, sizeof(extra));
    if (int rc = launch_raw(m, "keops_chk_knn_ymax", 1, 1, 256, buf.data(), psize + sizeof(extra), stream)) return rc;
    if (int rc = launch_raw(m, "keops_chk_knn_rerank", (unsigned)((nx + 3) / 4), 1, 256, buf.data(), psize + sizeof(extra), stream)) return rc;
    if (int rc = ensure_pinned(m, 64)) return rc;
    HIP_TRY(hipMemcpyAsync(m.pinned, ws + o_flag, 4, hipMemcpyDeviceToHost, stream));
    HIP_TRY(hipStreamSynchronize(stream));
    const int bad = *(volatile int*)m.pinned;
    if (bad != 0)
      return fail(KEOPS_HIP_NOT_CERTIFIED, std::to_string(bad) + " rows have neighbours that the matrix-core pass cannot separate "
                                           "(ties or near-ties at the K-th distance): recompute this call on the exact kernel");
  }
  return 0;
}

// ---- float64 matrix-core chunked scheme (kernels/keops_chunk_f64.h) --------------------------------

// must match struct C64Params of kernels/keops_chunk_f64.h (argument pointers follow)
struct C64Header {
  int64_t nx, ny;
  void* xs;
  void* ys;
  void* xn;
  void* yn;
  void* colsum;
  void* colpart;
  void* out;
  int64_t nxs, nys;
  RangeHeader rt;
};

int launch_chunk64(Module& m, int64_t nx, int64_t ny, void* out, void* const* args, hipStream_t stream, const RangeLaunch* rg,
                   int64_t nxs, int64_t nys) {
  const int64_t D = m.meta_int("chk_d", 0), DP = m.meta_int("chk_dpad", 0), QB = m.meta_int("chk_qb", 128);
  const int mode = m.meta_int("chk_mode", 0);
  if (D <= 0 || DP <= 0 || DP % 8 != 0) return fail(-1, "corrupt chunk module metadata");
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off = align_up(off + bytes, 256); return o; };
  const int nparts = (int)std::max<int64_t>(1, std::min<int64_t>(256, nys / 64));
  const size_t o_colsum = take((size_t)DP * 8), o_colpart = take((size_t)nparts * DP * 8);
  const size_t o_xs = take((size_t)nxs * DP * 8), o_ys = take((size_t)nys * DP * 8);
  const size_t o_xn = take((size_t)nxs * 8), o_yn = take((size_t)nys * 8);
  if (int rc = m.partial.reserve(off)) return rc;
  char* ws = (char*)m.partial.ptr;
  const int64_t row_blocks = rg ? rg->tables.nblocks : (nx + QB - 1) / QB;
  std::vector<char> buf(sizeof(C64Header) + sizeof(void*) * (size_t)std::max(1, m.nargs) + 32);
  C64Header h{};
  h.nx = nx; h.ny = ny; h.xs = ws + o_xs; h.ys = ws + o_ys; h.xn = ws + o_xn; h.yn = ws + o_yn; h.colsum = ws + o_colsum;
  h.colpart = ws + o_colpart; h.out = out; h.nxs = nxs; h.nys = nys;
  if (rg) h.rt = rg->header(m.nargs);
  std::memcpy(buf.data(), &h, sizeof(h));
  for (int k = 0; k < m.nargs; k++) std::memcpy(buf.data() + sizeof(h) + sizeof(void*) * k, &args[k], sizeof(void*));
  const size_t psize = sizeof(C64Header) + sizeof(void*) * (size_t)std::max(1, m.nargs);
  int32_t which = 0;
  auto with_which = [&](int w) { which = w; std::memcpy(buf.data() + psize, &which, 4); return psize + 4; };
  if (mode == 0) {
    if (int rc = launch_raw(m, "keops_c64_colsum", (unsigned)nparts, 1, 256, buf.data(), psize, stream)) return rc;
    const size_t szp = with_which(nparts);
    if (int rc = launch_raw(m, "keops_c64_colsum_final", 1, 1, 256, buf.data(), szp, stream)) return rc;
  }
  size_t sz = with_which(0);
  if (int rc = launch_raw(m, "keops_c64_prep", (unsigned)((nxs * 8 + 255) / 256), 1, 256, buf.data(), sz, stream)) return rc;
  sz = with_which(1);
  if (int rc = launch_raw(m, "keops_c64_prep", (unsigned)((nys * 8 + 255) / 256), 1, 256, buf.data(), sz, stream)) return rc;
  if (rg && rg->user_ranges)
    if (int rc = launch_raw(m, "keops_c64_fill_neutral", (unsigned)((nx + 255) / 256), 1, 256, buf.data(), psize, stream)) return rc;
  if (m.timing) HIP_TRY(hipEventRecord(m.ev0, stream));
  if (int rc = launch_raw(m, "keops_c64_main", (unsigned)row_blocks, 1, (unsigned)m.block, buf.data(), psize, stream)) return rc;
  if (m.timing) HIP_TRY(hipEventRecord(m.ev1, stream));
  return 0;
}

// ---- matrix-core final-product scheme (kernels/keops_final_mfma.h) ----------------------------------

// must match struct FinParams of kernels/keops_final_mfma.h (argument pointers follow)
struct FinHeader {
  int64_t nx, ny;
  void* out;
  void* partial;
  int64_t slab_len;
  int32_t nslabs;
  int32_t pad_;
  void* vsplit;
  int64_t vrows;
  RangeHeader rt;
};

// vrows: rows of the array v (with batch dimensions: of all its batches; else the reduced size)
int launch_final(Module& m, int64_t nx, int64_t ny, void* out, void* const* args, int tag1D2D, hipStream_t stream,
                 const RangeLaunch* rg, int64_t vrows) {
  const int64_t DV = m.meta_int("fin_dv", 0), NZ = m.meta_int("fin_nz", 1), QB = m.meta_int("fin_qb", 256), TJ = m.tile_j;
  if (DV <= 0 || NZ <= 0 || QB <= 0 || TJ <= 0) return fail(-1, "corrupt final-product module metadata");
  const int64_t row_blocks = rg ? rg->tables.nblocks : (nx + QB - 1) / QB;
  // enough workgroups for the chip: cut the reduced axis in slabs when there are few output rows
  int64_t nslabs = 1;
  const int64_t target = 2 * (int64_t)m.cu_count;
  if (!rg && (tag1D2D == 1 || row_blocks * NZ < target)) {
    const int64_t max_slabs = std::max<int64_t>(1, ny / (8 * TJ));
    nslabs = std::min<int64_t>(max_slabs, (target + row_blocks * NZ - 1) / (row_blocks * NZ));
    if (tag1D2D == 1) nslabs = std::max<int64_t>(nslabs, std::min<int64_t>(max_slabs, 2));
    nslabs = std::max<int64_t>(1, std::min<int64_t>(nslabs, 65535));
  }
  // one workgroup (8 wavefronts of ~230 VGPRs) fills a CU and all of them take the same time
  if (!rg) nslabs = balance_slabs(row_blocks * NZ, nslabs, std::min<int64_t>(std::max<int64_t>(nslabs, 8), std::max<int64_t>(1, ny / (8 * TJ))), m.cu_count);
  int64_t len = std::max<int64_t>(TJ, ((ny + nslabs - 1) / nslabs + TJ - 1) / TJ * TJ);
  nslabs = std::max<int64_t>(1, (ny + len - 1) / len);
  FinHeader h{};
  h.nx = nx; h.ny = ny; h.out = out; h.slab_len = len; h.nslabs = (int32_t)nslabs;
  if (rg) h.rt = rg->header(m.nargs);
  // split-operand variant: v rewritten once as three bfloat16 terms, tile by tile (tiles are counted along the
  // array v, whatever the ranges and batches of the launch)
  const bool split3 = m.meta_int("fin_split3", 0) != 0;
  h.vrows = vrows;
  const int64_t DVP = (DV + 31) / 32 * 32, ntiles = (vrows + TJ - 1) / TJ;
  // sums kept in double (meta fin_acc64): the folds always go to the partial buffer, keops_fin_reduce rounds once
  const bool acc64 = m.meta_int("fin_acc64", 0) != 0;
  if (acc64 && rg) return fail(-1, "corrupt final-product module metadata");
  const size_t part_bytes = (nslabs > 1 || acc64) ? align_up((size_t)nslabs * nx * DV * (acc64 ? 8 : 4), 256) : 0;
  const size_t split_bytes = split3 ? (size_t)ntiles * 3 * DVP * TJ * 2 : 0;
  if (part_bytes + split_bytes > 0) {
    if (int rc = m.partial.reserve(part_bytes + split_bytes)) return rc;
    if (nslabs > 1 || acc64) h.partial = m.partial.ptr;
    if (split3) h.vsplit = (char*)m.partial.ptr + part_bytes;
  }
  std::vector<char> buf(sizeof(FinHeader) + sizeof(void*) * (size_t)std::max(1, m.nargs));
  std::memcpy(buf.data(), &h, sizeof(h));
  for (int k = 0; k < m.nargs; k++) std::memcpy(buf.data() + sizeof(h) + sizeof(void*) * k, &args[k], sizeof(void*));
  if (rg && rg->user_ranges)
    if (int rc = launch_raw(m, "keops_fin_fill_neutral", (unsigned)((nx * DV + 255) / 256), 1, 256, buf.data(), buf.size(), stream)) return rc;
  if (split3)
    if (int rc = launch_raw(m, "keops_fin_split", (unsigned)((ntiles * DVP * TJ + 255) / 256), 1, 256, buf.data(), buf.size(), stream)) return rc;
  if (m.timing) HIP_TRY(hipEventRecord(m.ev0, stream));
  if (int rc = launch_raw3(m, split3 ? "keops_fin_main3" : "keops_fin_main", (unsigned)row_blocks, (unsigned)nslabs, (unsigned)NZ, (unsigned)m.block, buf.data(), buf.size(), stream)) return rc;
  if (m.timing) HIP_TRY(hipEventRecord(m.ev1, stream));
  if (nslabs > 1 || acc64) {
    const int64_t gb = (nx * DV + 255) / 256;
    if (int rc = launch_raw(m, "keops_fin_reduce", (unsigned)gb, 1, 256, buf.data(), buf.size(), stream)) return rc;
  }
  return 0;
}

}  // namespace

// =================================================================================================

extern "C" {

int keops_hip_abi_version(void) { return 3; }

const char* keops_hip_templates_digest(void) { return keops_templates_digest; }

int keops_hip_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return n;
}

const char* keops_hip_last_error(void) { return g_last_error.c_str(); }

int keops_hip_compile(const char* target_file, const char* hip_src, int use_fast_math, int device_id) {
  if (!target_file || !hip_src) return fail(-1, "keops_hip_compile: null argument");
  std::vector<const char*> hdr_text, hdr_name;
  for (const EmbeddedHeader* h = keops_embedded_headers; h->name; ++h) {
    hdr_name.push_back(h->name);
    hdr_text.push_back(h->text);
  }
  hiprtcProgram prog;
  hiprtcResult r = hiprtcCreateProgram(&prog, hip_src, "keops_module.hip", (int)hdr_name.size(), hdr_text.data(), hdr_name.data());
  if (r != HIPRTC_SUCCESS) return fail((int)r, std::string("hiprtcCreateProgram: ") + hiprtcGetErrorString(r));
  const std::string arch = "--offload-arch=" + target_arch(device_id);
  // optimisation level: -O3 unless KEOPS_HIP_OPT_LEVEL names another one (very long straight-line kernels)
  const char* lvl = getenv("KEOPS_HIP_OPT_LEVEL");
  const std::string olevel = std::string("-O") + (lvl && *lvl ? lvl : "3");
  std::vector<const char*> opts = {arch.c_str(), olevel.c_str(), "-std=c++17", "-fno-math-errno", "-ffp-contract=fast-honor-pragmas",
                                   // packed FP32 instructions are kept out of every kernel of this library
                                   "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
  const std::string fm = std::string("-DKEOPS_FAST_MATH=") + (use_fast_math ? "1" : "0");
  opts.push_back(fm.c_str());
  r = hiprtcCompileProgram(prog, (int)opts.size(), opts.data());
  if (r != HIPRTC_SUCCESS) {
    size_t n = 0;
    hiprtcGetProgramLogSize(prog, &n);
    std::string log(n, '\0');
    if (n) hiprtcGetProgramLog(prog, &log[0]);
    hiprtcDestroyProgram(&prog);
    return fail((int)r, std::string("hiprtc compilation failed (") + hiprtcGetErrorString(r) + "):\n" + log);
  }
  size_t n = 0;
  hiprtcGetCodeSize(prog, &n);
  std::vector<char> code(n);
  hiprtcGetCode(prog, code.data());
  hiprtcDestroyProgram(&prog);

  const std::string meta = collect_meta(hip_src);
  const std::string tmp = std::string(target_file) + ".tmp" + std::to_string((long)getpid());
  {
    std::ofstream out(tmp, std::ios::binary);
    if (!out) return fail(-1, "cannot write " + tmp);
    uint64_t cs = code.size(), ms = meta.size();
    out.write((const char*)&cs, sizeof(cs));
    out.write(code.data(), (std::streamsize)cs);
    out.write((const char*)&ms, sizeof(ms));
    out.write(meta.data(), (std::streamsize)ms);
  }
  if (std::rename(tmp.c_str(), target_file) != 0) return fail(-1, std::string("cannot rename to ") + target_file);
  return 0;
}

void* keops_hip_module_create(int device_id, int nargs, const char* target_file) {
  std::ifstream in(target_file, std::ios::binary);
  if (!in) {
    fail(-1, std::string("cannot open module file ") + target_file);
    return nullptr;
  }
  uint64_t cs = 0, ms = 0;
  in.read((char*)&cs, sizeof(cs));
  std::vector<char> code(cs);
  in.read(code.data(), (std::streamsize)cs);
  in.read((char*)&ms, sizeof(ms));
  std::string meta(ms, '\0');
  if (ms) in.read(&meta[0], (std::streamsize)ms);
  if (!in) {
    fail(-1, std::string("truncated module file ") + target_file);
    return nullptr;
  }
  Module* m = new Module();
  m->device = device_id < 0 ? 0 : device_id;
  m->nargs = nargs;
  m->meta = parse_meta(meta);
  hipError_t e = hipSetDevice(m->device);
  if (e == hipSuccess) e = hipModuleLoadData(&m->mod, code.data());
  if (e != hipSuccess) {
    fail((int)e, std::string("loading module on device ") + std::to_string(m->device) + " failed: " + hipGetErrorString(e));
    delete m;
    return nullptr;
  }
  {
    // The library's own device code (fill, conversion and range-table kernels, the static scratch array) is loaded
    // on a device at its first use, which takes about 50 ms (the array is 128 MiB): here, once per device, rather
    // than inside some later launch -- the second call of a block-sparse launch, or one under graph capture.
    void* sp = nullptr;
    size_t sb = 0;
    if (keops_static_scratch(m->device, &sp, &sb) != 0) (void)hipGetLastError();
  }
  int cus = 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, m->device) == hipSuccess && cus > 0) m->cu_count = cus;
  m->block = m->meta_int("block", 256);
  m->rows = m->meta_int("rows", 1);
  m->tile_j = m->meta_int("tile_j", 256);
  m->dimred = m->meta_int("dimred", 1);
  m->dimout = m->meta_int("dimout", 1);
  m->sizeof_t = m->meta_int("sizeof_t", 4);
  m->sizeof_acc = m->meta_int("sizeof_acc", 4);
  m->nrowvars = m->meta_int("nrowvars", 0);
  m->ncolvars = m->meta_int("ncolvars", 0);
  m->nparvars = m->meta_int("nparvars", 0);
  m->scheme = m->meta.count("scheme") ? m->meta["scheme"] : "conv";
  return m;
}

void keops_hip_module_destroy(void* module) {
  Module* m = (Module*)module;
  if (!m) return;
  (void)hipSetDevice(m->device);
  if (m->tables_in_flight && m->tables_copied) (void)hipEventSynchronize(m->tables_copied);
  m->partial.release();
  m->tables.release();
  m->staging.release();
  if (m->last_done) (void)hipEventDestroy(m->last_done);
  if (m->pinned) (void)hipHostFree(m->pinned);
  // (the status words are not read here: at interpreter exit the runtime may already have unmapped pinned memory)
  if (m->ranges_status) (void)hipHostFree(m->ranges_status);
  for (void* p : m->retired_pinned) (void)hipHostFree(p);
  if (m->tables_copied) (void)hipEventDestroy(m->tables_copied);
  if (m->ev0) (void)hipEventDestroy(m->ev0);
  if (m->ev1) (void)hipEventDestroy(m->ev1);
  if (m->mod) (void)hipModuleUnload(m->mod);
  delete m;
}

const char* keops_hip_module_meta(void* module, const char* key) {
  Module* m = (Module*)module;
  if (!m || !key) return nullptr;
  auto it = m->meta.find(key);
  return it == m->meta.end() ? nullptr : it->second.c_str();
}

void keops_hip_module_set_timing(void* module, int enabled) {
  Module* m = (Module*)module;
  if (m) m->timing = enabled != 0;
}

double keops_hip_module_last_kernel_ms(void* module) {
  Module* m = (Module*)module;
  return m ? m->last_ms : -1.0;
}

// One map-reduce on device-resident arguments (the body of keops_hip_launch).
static int launch_on_device(Module& m, int64_t nx, int64_t ny, int tagI, int tagZero, int tag1D2D, int64_t dimred,
                            const int* indsi, int ni, const int* indsj, int nj, const int* indsp, int np,
                            int64_t dimout, const int64_t* dimsx, const int64_t* dimsy, const int64_t* dimsp,
                            int64_t* const* ranges, const int64_t* shapeout, int nshapeout, void* out,
                            void* const* args, const int64_t* argshapes_flat, const int* argndims,
                            hipStream_t stream, int sync) {
  if (dimred != m.dimred || dimout != m.dimout)
    return fail(-1, "dimred/dimout do not match the compiled module");

  int64_t sizeout = 1;
  for (int k = 0; k < nshapeout; k++) sizeout *= shapeout[k];

  if (tagZero) {
    // a fill kernel, not hipMemsetAsync: the launch may be recorded into a HIP graph
    if (int e = keops_static_fill_zero(out, (size_t)sizeout * m.sizeof_t, stream))
      return fail(e, std::string("zero fill failed: ") + hipGetErrorString((hipError_t)e));
    if (sync) HIP_TRY(hipStreamSynchronize(stream));
    return 0;
  }

  // The workspaces and tables of a module are shared by all its launches.  (1) Once a launch has been recorded
  // into a HIP graph they keep their address and contents (the graph holds raw pointers into them); (2) a launch
  // on another stream than the previous one first waits for it.
  const bool capturing = stream_is_capturing(stream);
  if (capturing && !m.captured) {
    m.captured = true;
  }
  if (capturing) {
    m.partial.frozen = m.tables.frozen = true;
    m.pinned_frozen = true;
  }
  if (!capturing && m.has_last && m.last_stream != stream) HIP_TRY(hipStreamWaitEvent(stream, m.last_done, 0));

  // ---- shapes (Sizes.h) ----
  std::vector<int> vI(indsi, indsi + ni), vJ(indsj, indsj + nj), vP(indsp, indsp + np);
  std::vector<int64_t> dX(dimsx, dimsx + ni), dY(dimsy, dimsy + nj), dP(dimsp, dimsp + np);
  std::vector<std::vector<int64_t>> argshapes(m.nargs);
  {
    const int64_t* p = argshapes_flat;
    for (int k = 0; k < m.nargs; k++) {
      argshapes[k].assign(p, p + argndims[k]);
      p += argndims[k];
    }
  }
  ShapeTable S;
  std::string err;
  if (int rc = S.build(m.nargs, argshapes, nx, ny, dimout, vI, vJ, vP, dX, dY, dP, err)) return fail(rc, err);
  const int nb = S.nbatchdims;
  const int64_t NX = S.nbatches * S.M, NY = S.nbatches * S.N;

  // the kernel's "rows" are the output-indexed variables, its "columns" the reduced ones
  const int64_t rows_total = tagI == 0 ? NX : NY;
  const int64_t cols_total = tagI == 0 ? NY : NX;
  const std::vector<int>& rowvars = tagI == 0 ? vI : vJ;
  const std::vector<int>& colvars = tagI == 0 ? vJ : vI;
  if ((int)rowvars.size() != m.nrowvars || (int)colvars.size() != m.ncolvars || (int)vP.size() != m.nparvars)
    return fail(-1, "variable lists do not match the compiled module");
  if (sizeout != rows_total * dimout)
    return fail(-1, "output has " + std::to_string(sizeout) + " elements, expected " + std::to_string(rows_total * dimout));
  if (rows_total == 0) return 0;

  const bool user_ranges = ranges && ranges[6] && ranges[6][0] != -1;
  if (user_ranges && nb > 0)
    return fail(-1, "the 'ranges' argument (block-sparse mode) is not supported with batch processing");
  const bool use_ranges = user_ranges || nb > 0;
  const int64_t rows_per_block = (int64_t)m.block * m.rows;

  if (m.timing) {
    if (!m.ev0) { HIP_TRY(hipEventCreate(&m.ev0)); HIP_TRY(hipEventCreate(&m.ev1)); }
  }
  if (g_noalloc && (user_ranges || nb > 0))
    return fail(-1, "keops_hip_launch_noalloc: block-sparse and batched launches build device tables; use keops_hip_launch");
  m.last_ms = -1.0;

  LaunchHeader h{};
  h.nx = rows_total;
  h.ny = cols_total;
  h.out = out;
  h.nbatchdims = nb;
  h.nslabs = 1;
  h.slab_len = cols_total;

  // nothing to reduce over: every output row is the reduction's neutral element (a sum of no terms, the log-sum-exp
  // pair (-inf, 0), +inf for a minimum ...), as the reference's loops leave it
  if (cols_total == 0) {
    if (m.scheme != "conv")
      return fail(-1, "the reduced axis is empty: only the general-purpose module (enable_chunks = 0) serves such a call");
    const int64_t gb = (rows_total + m.block - 1) / m.block;
    if (int rc = launch(m, "keops_fill_neutral", (unsigned)gb, 1, h, args, stream)) return rc;
    if (sync) HIP_TRY(hipStreamSynchronize(stream));
    return 0;
  }

  if (m.scheme == "knn") {
    const bool built_for_ranges = m.meta_int("ranges", 0) != 0;
    const int rowarg = m.meta_int("rowarg", 0), colarg = m.meta_int("colarg", 1);
    if (rowarg < 0 || colarg < 0 || rowarg >= m.nargs || colarg >= m.nargs) return fail(-1, "corrupt knn module metadata");
    // many batches on a module built for ranges: every batch is one row range with one reduced-index range, provided
    // queries and references carry every batch dimension in full (no broadcasting)
    bool batches_as_ranges = false;
    if (built_for_ranges && nb > 0 && !user_ranges) {
      auto full = [&](int arg) {
        const int64_t* r = S.row(arg + 1);
        for (int b = 0; b < nb; b++)
          if (r[b] != S.shapes[b]) return false;
        return true;
      };
      if (!full(rowarg) || !full(colarg))
        return fail(-1, "this K-nearest-neighbour module serves batches as row ranges: queries and references must carry "
                        "every batch dimension (no broadcasting)");
      batches_as_ranges = true;
    }
    if (!batches_as_ranges && (user_ranges != built_for_ranges || (built_for_ranges && nb > 0)))
      return fail(-1, built_for_ranges ? "this K-nearest-neighbour module was built for block-sparse ranges without batch dimensions"
                                       : "this K-nearest-neighbour module does not handle block-sparse ranges");
    if (batches_as_ranges) {
      RangeLaunch rg;
      rg.nbatchdims = 0;  // rows are addressed globally: the kernel sees plain ranges over the flattened batches
      rg.user_ranges = false;
      if (int rc = prepare_range_tables(m, S, tagI, false, ranges, rows_total, cols_total, m.meta_int("knn_qb", 256), true, rowvars,
                                        colvars, vP, stream, rg.tables))
        return rc;
      rg.tables.offsets = nullptr;
      const int64_t R = tagI == 0 ? S.M : S.N, C = tagI == 0 ? S.N : S.M;
      if (int rc = launch_knn_ranges(m, rows_total, cols_total, args[rowarg], args[colarg], out, stream, rg, R, C)) return rc;
    } else if (user_ranges) {
      RangeLaunch rg;
      rg.nbatchdims = 0;
      rg.user_ranges = true;
      if (int rc = prepare_range_tables(m, S, tagI, true, ranges, rows_total, cols_total, m.meta_int("knn_qb", 256), true, rowvars,
                                        colvars, vP, stream, rg.tables))
        return rc;
      if (int rc = launch_knn_ranges(m, rows_total, cols_total, args[rowarg], args[colarg], out, stream, rg)) return rc;
    } else if (nb == 0) {
      if (int rc = launch_knn(m, rows_total, cols_total, args[rowarg], args[colarg], out, tag1D2D, stream)) return rc;
    } else {
      // batch dimensions: one pass of the dense pipeline per batch on the same stream (indices are relative to
      // the batch, as in GpuReduc1D_ranges.py:151-158); a batch dimension of size 1 is broadcast
      const int64_t R = tagI == 0 ? S.M : S.N, C = tagI == 0 ? S.N : S.M;
      const int64_t D = m.meta_int("knn_d", 0);
      std::vector<int64_t> shp(nb + 1);
      auto first_row = [&](int arg, int64_t b, int64_t len) {
        const int64_t* r = S.row(arg + 1);
        for (int k = 0; k < nb; k++) shp[k] = r[k];
        shp[nb] = len;
        return broadcast_index(b * len, nb, S.shapes.data(), shp.data());
      };
      const bool timing = m.timing;
      if (timing) HIP_TRY(hipEventRecord(m.ev0, stream));
      m.timing = false;
      int rc = 0;
      for (int64_t b = 0; b < S.nbatches && rc == 0; b++) {
        const char* xq = (const char*)args[rowarg] + first_row(rowarg, b, R) * D * m.sizeof_t;
        const char* yr = (const char*)args[colarg] + first_row(colarg, b, C) * D * m.sizeof_t;
        rc = launch_knn(m, R, C, xq, yr, (char*)out + b * R * dimout * m.sizeof_t, tag1D2D, stream);
      }
      m.timing = timing;
      if (rc) return rc;
      if (timing) HIP_TRY(hipEventRecord(m.ev1, stream));
    }
  } else if (m.scheme == "final" || m.scheme == "chunk" || m.scheme == "chunk64") {
    const bool built_for_ranges = m.meta_int("ranges", 0) != 0;
    if (use_ranges != built_for_ranges)
      return fail(-1, built_for_ranges ? "this module was built for block-sparse or batched reductions"
                                       : "this module was built for dense reductions without batch dimensions");
    RangeLaunch rg;
    if (use_ranges) {
      rg.nbatchdims = nb;
      rg.user_ranges = user_ranges;
      const int64_t qb = m.meta_int(m.scheme == "final" ? "fin_qb" : "chk_qb", 256);
      if (int rc = prepare_range_tables(m, S, tagI, user_ranges, ranges, rows_total, cols_total, qb, true, rowvars, colvars, vP, stream,
                                        rg.tables))
        return rc;
    }
    // rows of an argument: a batch dimension of size 1 is broadcast, not stored
    auto arg_rows = [&](int arg, int64_t len) {
      const int64_t* r = S.row(arg + 1);
      int64_t n = len;
      for (int b = 0; b < nb; b++) n *= r[b];
      return n;
    };
    if (m.scheme == "final") {
      const int varg = m.meta_int("fin_varg", -1);
      if (varg < 0 || varg >= m.nargs) return fail(-1, "corrupt final-product module metadata");
      const int64_t vrows = nb > 0 ? arg_rows(varg, tagI == 0 ? S.N : S.M) : cols_total;
      if (int rc = launch_final(m, rows_total, cols_total, out, args, tag1D2D, stream, use_ranges ? &rg : nullptr, vrows)) return rc;
    } else {
      const int xarg = m.meta_int("chk_xarg", -1), yarg = m.meta_int("chk_yarg", -1);
      if (xarg < 0 || yarg < 0 || xarg >= m.nargs || yarg >= m.nargs) return fail(-1, "corrupt chunk module metadata");
      const int64_t nxs = nb > 0 ? arg_rows(xarg, tagI == 0 ? S.M : S.N) : rows_total;
      const int64_t nys = nb > 0 ? arg_rows(yarg, tagI == 0 ? S.N : S.M) : cols_total;
      if (m.scheme == "chunk64") {
        if (int rc = launch_chunk64(m, rows_total, cols_total, out, args, stream, use_ranges ? &rg : nullptr, nxs, nys)) return rc;
      } else if (int rc = launch_chunk(m, rows_total, cols_total, out, args, tag1D2D, stream, use_ranges ? &rg : nullptr, nxs, nys))
        return rc;
    }
  } else if (!use_ranges) {
    // ---- dense scheme, optionally cut in column slabs ----
    const int64_t row_blocks = (rows_total + rows_per_block - 1) / rows_per_block;
    int64_t nslabs = 1;
    // many short slabs: with few rows every SIMD still holds several wavefronts to hide the latency of the
    // dependent per-pair chain, and with many rows the fine-grained grid keeps all CUs busy to the end
    // (1e6 x 1e6 Gaussian sum: 226 ms with one slab, 187 ms with 17)
    static const int64_t per_cu = [] {
      const char* e = std::getenv("KEOPS_HIP_BLOCKS_PER_CU");
      const int64_t v = e ? std::atoll(e) : 0;
      return v > 0 ? v : (int64_t)64;
    }();
    // K-smallest lists restart empty in every slab (more insertions, 2K values per row and slab to merge):
    // fewer, longer slabs for that family
    const int64_t target_blocks = (m.meta_int("red_kind", 0) == 4 ? std::min<int64_t>(per_cu, 8) : per_cu) * (int64_t)m.cu_count;
    if (tag1D2D == 1 || row_blocks * 2 <= target_blocks) {
      const int64_t max_slabs = std::max<int64_t>(1, cols_total / 256);
      nslabs = std::min<int64_t>(max_slabs, (target_blocks + row_blocks - 1) / row_blocks);
      if (tag1D2D == 1) nslabs = std::max<int64_t>(nslabs, std::min<int64_t>(max_slabs, 2));
      nslabs = std::min<int64_t>(nslabs, 65535);
      // the per-slab partial accumulators stay within 256 MB
      const int64_t row_bytes = std::max<int64_t>(1, rows_total * m.dimred * m.sizeof_acc);
      nslabs = std::min<int64_t>(nslabs, std::max<int64_t>(tag1D2D == 1 ? 2 : 1, (256LL << 20) / row_bytes));
    }
    if (nslabs > 1) {
      int64_t len = (cols_total + nslabs - 1) / nslabs;
      len = ((len + 63) / 64) * 64;
      nslabs = (cols_total + len - 1) / len;
      h.slab_len = len;
    }
    h.nslabs = (int32_t)nslabs;
    const size_t slab_bytes = nslabs > 1 ? (size_t)nslabs * rows_total * m.dimred * m.sizeof_acc : 0;
    const bool radial = m.meta_int("radial", 0) != 0;
    if (radial) {
      // exponents on the matrix cores when the data allow it (decided on the device); the kernels below then return
      // at once, and the other way round.  Both share the workspace: slab partials first.
      if (int rc = launch_radial(m, rows_total, cols_total, out, args, stream, slab_bytes, &h.guard)) return rc;
      m.last_guard = h.guard;
    } else if (slab_bytes) {
      if (int rc = m.partial.reserve(slab_bytes)) return rc;
    }
    if (nslabs > 1) h.partial = m.partial.ptr;
    if (m.timing && !radial) HIP_TRY(hipEventRecord(m.ev0, stream));
    if (int rc = launch(m, "keops_conv_dense", (unsigned)row_blocks, (unsigned)nslabs, h, args, stream)) return rc;
    if (m.timing) HIP_TRY(hipEventRecord(m.ev1, stream));
    if (nslabs > 1) {
      const int64_t gb = (rows_total + m.block - 1) / m.block;
      if (int rc = launch(m, "keops_reduce_partials", (unsigned)gb, 1, h, args, stream)) return rc;
    }
  } else {
    // ---- block-sparse / batched scheme (Ranges.h, keops_nvrtc.cpp:152-248) ----
    RangeTables rt;
    if (int rc = prepare_range_tables(m, S, tagI, user_ranges, ranges, rows_total, cols_total, rows_per_block, false, rowvars, colvars,
                                      vP, stream, rt))
      return rc;
    const int64_t nblocks = rt.nblocks;
    h.lookup = rt.lookup;
    h.offsets = rt.offsets;
    h.slices_x = rt.slices_x;
    h.ranges_y = rt.ranges_y;
    if (m.timing) HIP_TRY(hipEventRecord(m.ev0, stream));
    if (user_ranges) {
      const int64_t gb = (rows_total + m.block - 1) / m.block;
      if (int rc = launch(m, "keops_fill_neutral", (unsigned)gb, 1, h, args, stream)) return rc;
      // exponents on the matrix cores when the pattern and the data allow it (the latter is decided on the device):
      // keops_conv_ranges then returns at once, and the other way round
      if (m.meta_int("radial", 0) != 0 && m.meta_int("rad_ranges", 0) != 0)
        if (int rc = launch_radial_ranges(m, rows_total, cols_total, out, args, stream, rt, &h.guard)) return rc;
      m.last_guard = h.guard;
    } else if (m.meta_int("radial", 0) != 0 && m.meta_int("rad_ranges", 0) != 0) {
      // batches: row ranges over the flattened arrays when every row and column variable carries every batch
      // dimension and no parameter does (the kernels of that family address rows globally and read one parameter set)
      bool plain = true;
      for (int v : rowvars) { const int64_t* r = S.row(v + 1); for (int b = 0; b < nb; b++) plain = plain && r[b] == S.shapes[b]; }
      for (int v : colvars) { const int64_t* r = S.row(v + 1); for (int b = 0; b < nb; b++) plain = plain && r[b] == S.shapes[b]; }
      for (int v : vP) { const int64_t* r = S.row(v + 1); for (int b = 0; b < nb; b++) plain = plain && r[b] == 1; }
      if (plain)
        if (int rc = launch_radial_ranges(m, rows_total, cols_total, out, args, stream, rt, &h.guard)) return rc;
      m.last_guard = h.guard;
    }
    if (int rc = launch(m, "keops_conv_ranges", (unsigned)nblocks, 1, h, args, stream)) return rc;
    if (m.timing) HIP_TRY(hipEventRecord(m.ev1, stream));
  }

  if (m.timing) {
    HIP_TRY(hipEventSynchronize(m.ev1));
    float ms = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, m.ev0, m.ev1));
    m.last_ms = ms;
  }
  if (!capturing) {
    if (!m.last_done && !g_noalloc) HIP_TRY(hipEventCreateWithFlags(&m.last_done, hipEventDisableTiming));
    if (m.last_done) {
      HIP_TRY(hipEventRecord(m.last_done, stream));
      m.last_stream = stream;
      m.has_last = true;
    }
  }
  if (sync) HIP_TRY(hipStreamSynchronize(stream));
  return 0;
}

// Host-resident arguments (tagHostDevice = 0), the counterpart of load_args_FromHost and
// range_preprocess_from_host (keopscore/keopscore/include/utils_pe.h:66-99, binders/nvrtc/keops_nvrtc.cpp:250-325):
// one pooled device allocation owned by the module holds copies of the arguments, of the ranges and of out; the
// copies travel on the launch stream and the call returns once out is back in host memory.
static int launch_from_host(Module& m, int64_t nx, int64_t ny, int tagI, int tagZero, int tag1D2D, int64_t dimred,
                            const int* indsi, int ni, const int* indsj, int nj, const int* indsp, int np,
                            int64_t dimout, const int64_t* dimsx, const int64_t* dimsy, const int64_t* dimsp,
                            int64_t* const* ranges, const int64_t* shapeout, int nshapeout, void* out,
                            void* const* args, const int64_t* argshapes_flat, const int* argndims, hipStream_t stream) {
  if (stream_is_capturing(stream)) return fail(-1, "host-resident arguments cannot be used while a HIP graph is being captured");
  int64_t sizeout = 1;
  for (int k = 0; k < nshapeout; k++) sizeout *= shapeout[k];
  if (sizeout < 0) return fail(-1, "negative output shape");
  std::vector<size_t> arg_bytes((size_t)m.nargs), arg_off((size_t)m.nargs);
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off = align_up(off + bytes, 256); return o; };
  {
    const int64_t* p = argshapes_flat;
    for (int k = 0; k < m.nargs; k++) {
      int64_t n = 1;
      for (int d = 0; d < argndims[k]; d++) {
        if (p[d] < 0) return fail(-1, "negative dimension in the shape of argument " + std::to_string(k));
        n *= p[d];
      }
      p += argndims[k];
      arg_bytes[k] = (size_t)n * m.sizeof_t;
      arg_off[k] = take(arg_bytes[k]);
    }
  }
  const size_t out_bytes = (size_t)sizeout * m.sizeof_t, out_off = take(out_bytes);
  const bool user_ranges = ranges && ranges[6] && ranges[6][0] != -1;
  size_t rg_off[6] = {}, rg_bytes[6] = {};
  if (user_ranges)
    for (int k = 0; k < 6; k++) {
      if (ranges[6][k] < 0) return fail(-1, "negative row count in the ranges");
      rg_bytes[k] = (size_t)ranges[6][k] * ((k % 3 == 1) ? 1 : 2) * sizeof(int64_t);  // slices: one entry per range
      rg_off[k] = take(rg_bytes[k]);
    }
  if (int rc = m.staging.reserve(std::max<size_t>(off, 256))) return rc;
  char* base = (char*)m.staging.ptr;
  std::vector<void*> dargs((size_t)std::max(1, m.nargs));
  for (int k = 0; k < m.nargs; k++) {
    dargs[k] = base + arg_off[k];
    if (arg_bytes[k]) HIP_TRY(hipMemcpyAsync(dargs[k], args[k], arg_bytes[k], hipMemcpyHostToDevice, stream));
  }
  int64_t* dranges[7] = {};
  if (user_ranges) {
    for (int k = 0; k < 6; k++) {
      dranges[k] = (int64_t*)(base + rg_off[k]);
      if (rg_bytes[k]) HIP_TRY(hipMemcpyAsync(dranges[k], ranges[k], rg_bytes[k], hipMemcpyHostToDevice, stream));
    }
    dranges[6] = ranges[6];
  }
  // (the ranges are host memory: validated on the host at every call, never through the device-built tables)
  g_host_ranges = true;
  const int rc_launch = launch_on_device(m, nx, ny, tagI, tagZero, tag1D2D, dimred, indsi, ni, indsj, nj, indsp, np, dimout, dimsx,
                                         dimsy, dimsp, user_ranges ? dranges : ranges, shapeout, nshapeout, base + out_off,
                                         dargs.data(), argshapes_flat, argndims, stream, 0);
  g_host_ranges = false;
  if (rc_launch) return rc_launch;
  if (out_bytes) HIP_TRY(hipMemcpyAsync(out, base + out_off, out_bytes, hipMemcpyDeviceToHost, stream));
  HIP_TRY(hipStreamSynchronize(stream));
  return 0;
}

// Half-precision data (use_half = 1; KeOps_module<TYPE>::launch_kernel's use_half, keops_nvrtc.cpp:390-400, and
// pykeops/pykeops/torch/half2_convert.py): out and the arguments are plain row-major arrays of IEEE half on the
// device.  The kernels of this library compute in float32: the arguments are converted into the module's staging
// buffer, the float32 module runs on those copies and the result is rounded to half once, at the end (the reference
// computes in half2 arithmetic; results here are at least as accurate).
static int launch_half(Module& m, int64_t nx, int64_t ny, int tagI, int tagZero, int tag1D2D, int64_t dimred,
                       const int* indsi, int ni, const int* indsj, int nj, const int* indsp, int np,
                       int64_t dimout, const int64_t* dimsx, const int64_t* dimsy, const int64_t* dimsp,
                       int64_t* const* ranges, const int64_t* shapeout, int nshapeout, void* out,
                       void* const* args, const int64_t* argshapes_flat, const int* argndims, hipStream_t stream, int sync) {
  if (m.sizeof_t != 4) return fail(-1, "use_half needs a module compiled for float (half data is computed in float32)");
  int64_t sizeout = 1;
  for (int k = 0; k < nshapeout; k++) sizeout *= shapeout[k];
  if (sizeout < 0) return fail(-1, "negative output shape");
  std::vector<int64_t> arg_n((size_t)m.nargs);
  std::vector<size_t> arg_off((size_t)m.nargs);
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off = align_up(off + bytes, 256); return o; };
  const int64_t* p = argshapes_flat;
  for (int k = 0; k < m.nargs; k++) {
    int64_t n = 1;
    for (int d = 0; d < argndims[k]; d++) {
      if (p[d] < 0) return fail(-1, "negative dimension in the shape of argument " + std::to_string(k));
      n *= p[d];
    }
    p += argndims[k];
    arg_n[k] = n;
    arg_off[k] = take((size_t)n * sizeof(float));
  }
  const size_t out_off = take((size_t)sizeout * sizeof(float));
  const bool capturing = stream_is_capturing(stream);
  if (capturing) m.staging.frozen = true;
  // the staging buffer is shared by all launches of the module: a launch on another stream first waits for the last one
  if (!capturing && m.has_last && m.last_stream != stream) HIP_TRY(hipStreamWaitEvent(stream, m.last_done, 0));
  if (int rc = m.staging.reserve(std::max<size_t>(off, 256))) return rc;
  char* base = (char*)m.staging.ptr;
  std::vector<void*> fargs((size_t)std::max(1, m.nargs));
  for (int k = 0; k < m.nargs; k++) {
    fargs[k] = base + arg_off[k];
    if (int e = keops_static_convert_half(fargs[k], args[k], arg_n[k], 1, stream))
      return fail(e, std::string("half -> float conversion failed: ") + hipGetErrorString((hipError_t)e));
  }
  g_half_data = true;
  const int rc_launch = launch_on_device(m, nx, ny, tagI, tagZero, tag1D2D, dimred, indsi, ni, indsj, nj, indsp, np, dimout, dimsx,
                                         dimsy, dimsp, ranges, shapeout, nshapeout, base + out_off, fargs.data(), argshapes_flat,
                                         argndims, stream, 0);
  g_half_data = false;
  if (rc_launch) return rc_launch;
  if (int e = keops_static_convert_half(out, base + out_off, sizeout, 0, stream))
    return fail(e, std::string("float -> half conversion failed: ") + hipGetErrorString((hipError_t)e));
  if (!capturing && m.last_done) HIP_TRY(hipEventRecord(m.last_done, stream));  // the conversion reads the staging buffer too
  if (sync) HIP_TRY(hipStreamSynchronize(stream));
  return 0;
}

int keops_hip_launch(void* module, int tagHostDevice, int64_t dimY, int64_t nx, int64_t ny, int tagI,
                     int tagZero, int use_half, int tag1D2D, int64_t dimred, int64_t block_size, int use_chunk_mode,
                     const int* indsi, int ni, const int* indsj, int nj, const int* indsp, int np,
                     int64_t dimout, const int64_t* dimsx, const int64_t* dimsy, const int64_t* dimsp,
                     int64_t* const* ranges, const int64_t* shapeout, int nshapeout, void* out,
                     void* const* args, const int64_t* argshapes_flat, const int* argndims,
                     void* hip_stream, int sync) {
  (void)dimY; (void)block_size; (void)use_chunk_mode;
  Module* mp = (Module*)module;
  if (!mp) return fail(-1, "keops_hip_launch: null module");
  Module& m = *mp;
  if (tagHostDevice != 0 && tagHostDevice != 1) return fail(-1, "tagHostDevice must be 0 (host pointers) or 1 (device pointers)");
  hipStream_t stream = (hipStream_t)hip_stream;
  HIP_TRY(hipSetDevice(m.device));
  if (use_half != 0 && use_half != 1) return fail(-1, "use_half must be 0 or 1");
  if (use_half) {
    if (tagHostDevice == 0) return fail(-1, "use_half takes device pointers (tagHostDevice = 1)");
    return launch_half(m, nx, ny, tagI, tagZero, tag1D2D, dimred, indsi, ni, indsj, nj, indsp, np, dimout, dimsx, dimsy, dimsp,
                       ranges, shapeout, nshapeout, out, args, argshapes_flat, argndims, stream, sync);
  }
  if (tagHostDevice == 0)
    return launch_from_host(m, nx, ny, tagI, tagZero, tag1D2D, dimred, indsi, ni, indsj, nj, indsp, np, dimout, dimsx, dimsy, dimsp,
                            ranges, shapeout, nshapeout, out, args, argshapes_flat, argndims, stream);
  return launch_on_device(m, nx, ny, tagI, tagZero, tag1D2D, dimred, indsi, ni, indsj, nj, indsp, np, dimout, dimsx, dimsy, dimsp,
                          ranges, shapeout, nshapeout, out, args, argshapes_flat, argndims, stream, sync);
}

int keops_hip_launch_noalloc(void* module, int64_t nx, int64_t ny, int tagI, int tag1D2D, int64_t dimred,
                             const int* indsi, int ni, const int* indsj, int nj, const int* indsp, int np,
                             int64_t dimout, const int64_t* dimsx, const int64_t* dimsy, const int64_t* dimsp,
                             const int64_t* shapeout, int nshapeout, void* out, void* const* args,
                             const int64_t* argshapes_flat, const int* argndims, void* hip_stream) {
  Module* mp = (Module*)module;
  if (!mp) return fail(-1, "keops_hip_launch_noalloc: null module");
  Module& m = *mp;
  if (m.scheme == "knn" || m.meta_int("chk_knn_inner", 0) > 0)
    return fail(-1, "keops_hip_launch_noalloc: the K-nearest-neighbour schemes read flags back through pinned host memory; "
                    "use keops_hip_launch");
  if (m.timing) return fail(-1, "keops_hip_launch_noalloc: switch kernel timing off (it creates events)");
  hipStream_t stream = (hipStream_t)hip_stream;
  HIP_TRY(hipSetDevice(m.device));
  void* sp = nullptr;
  size_t sbytes = 0;
  if (int e = keops_static_scratch(m.device, &sp, &sbytes))
    return fail(e, std::string("address of the static scratch buffer: ") + hipGetErrorString((hipError_t)e));
  // the module's workspace is, for this call, a view of the static scratch buffer; nothing else may be allocated
  DeviceBuffer view;
  view.ptr = sp;
  view.bytes = sbytes;
  view.borrowed = true;
  std::swap(m.partial, view);
  g_noalloc = true;
  int64_t no_ranges[1] = {-1};
  int64_t* rg[7] = {no_ranges, no_ranges, no_ranges, no_ranges, no_ranges, no_ranges, no_ranges};
  int rc = launch_on_device(m, nx, ny, tagI, 0, tag1D2D, dimred, indsi, ni, indsj, nj, indsp, np, dimout, dimsx, dimsy, dimsp, rg,
                            shapeout, nshapeout, out, args, argshapes_flat, argndims, stream, 0);
  g_noalloc = false;
  std::swap(m.partial, view);
  return rc;
}

int keops_hip_path_status(void* module, unsigned* taken) {
  if (!module || !taken) return fail(-1, "keops_hip_path_status: null argument");
  Module& m = *static_cast<Module*>(module);
  *taken = 0u;
  if (!m.last_guard) return 0;
  HIP_TRY(hipSetDevice(m.device));
  if (m.has_last) HIP_TRY(hipEventSynchronize(m.last_done));
  HIP_TRY(hipMemcpy(taken, m.last_guard, sizeof(unsigned), hipMemcpyDeviceToHost));
  return 0;
}

int keops_hip_ranges_status(void* module, unsigned* status) {
  if (!module || !status) return fail(-1, "keops_hip_ranges_status: null argument");
  Module& m = *static_cast<Module*>(module);
  *status = 0u;
  if (!m.ranges_status) return 0;
  HIP_TRY(hipSetDevice(m.device));
  if (m.has_last) HIP_TRY(hipEventSynchronize(m.last_done));
  *status = (m.ranges_status[0] ? 1u : 0u) | (m.ranges_status[1] ? 2u : 0u);
  m.ranges_status[0] = m.ranges_status[1] = 0u;  // read: the next launch starts clean
  return 0;
}

size_t keops_hip_noalloc_scratch_bytes(void) { return (size_t)KEOPS_STATIC_SCRATCH_BYTES; }

}  // extern "C"
