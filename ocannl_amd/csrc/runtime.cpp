// Runtime behind the C ABI: devices, the pool table, events, copies, hiprtc compilation, linking
// and launching.  Mirrors the responsibilities of the reference CUDA backend
// (arrayjit/lib/cuda_backend.ml) without sharing its structure: one HIP stream per device, slabs
// from hipMalloc, kernels from hiprtc modules plus the precompiled MFMA kernels of this library.
#include <atomic>
#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <sstream>
#include <string>
#include <vector>

#include "../../include/ocannl_hip.h"
#include "codegen.hpp"
#include "gemm.hpp"
#include "llir.hpp"
#include "plan.hpp"

using namespace ocannl;

namespace {

thread_local std::string g_last_error;

struct RuntimeError : std::runtime_error { using std::runtime_error::runtime_error; };

void hip_check(hipError_t e, const char* what) {
  if (e != hipSuccess) throw RuntimeError(std::string(what) + ": " + hipGetErrorString(e));
}

// Scratch memory for ocannl_hip_routine_run_static_scratch, the entry point that may not allocate:
// device memory that belongs to the loaded library itself.  Every GPU holds its own copy at its own
// address until the process ends; host code reaches it only through the pointer that
// hipGetSymbolAddress returns (ocannl_hip_device::static_scratch), never through this name.
constexpr uint64_t kStaticScratchBytes = OCANNL_HIP_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Zero fill as a kernel, for the path that callers may record into a HIP graph.  Exactly `bytes`
// bytes from `p` are cleared, wherever they start: a context node is packed at an offset aligned to
// its element size only and is followed by its neighbour in the pool, so the unaligned head and tail
// go out as single bytes and only the 16-byte aligned body as 16-byte stores.
__global__ void __launch_bounds__(256) fill_zero_kernel(unsigned char* p, uint64_t bytes) {
  const uint64_t addr = reinterpret_cast<uint64_t>(p);
  uint64_t head = (16 - (addr & 15)) & 15;
  if (head > bytes) head = bytes;
  const uint64_t n16 = (bytes - head) / 16, tail = bytes - head - n16 * 16;
  const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n16) reinterpret_cast<uint4*>(p + head)[i] = uint4{0, 0, 0, 0};
  if (i < head) p[i] = 0;
  if (i < tail) p[head + n16 * 16 + i] = 0;
}

}  // namespace

struct ocannl_hip_device {
  int ordinal = 0;
  hipStream_t stream = nullptr;
  hipStream_t side_stream = nullptr;   // second queue for contractions off the critical path (Phase::stream == 1)
  void* static_scratch = nullptr;   // this device's copy of `scratch` (hipGetSymbolAddress at device set-up)
  std::map<int, std::pair<void*, uint64_t>> pools;   // pool_id -> (base, size)
  uint64_t used = 0;
  uint64_t scratch_used = 0;
  int live_events = 0;
  int live_routines = 0;
  hipDeviceProp_t props{};
  void make_current() const { hip_check(hipSetDevice(ordinal), "hipSetDevice"); }
  void* resolve(int pool_id, uint64_t offset, uint64_t bytes, const char* what) const {
    auto it = pools.find(pool_id);
    if (it == pools.end()) throw InvalidArgument(std::string(what) + ": unknown pool_id " + std::to_string(pool_id));
    if (offset > it->second.second || bytes > it->second.second - offset)
      throw InvalidArgument(std::string(what) + ": range [" + std::to_string(offset) + ", +" + std::to_string(bytes) +
                            ") exceeds pool " + std::to_string(pool_id) + " of " + std::to_string(it->second.second) + " bytes");
    return static_cast<char*>(it->second.first) + offset;
  }
};

struct ocannl_hip_event {
  hipEvent_t ev = nullptr;
  ocannl_hip_device* dev = nullptr;
};

namespace {

struct CompiledRoutine {
  Routine r;
  Plan plan;
  GeneratedModule mod;
  std::vector<char> binary;   // gfx950 code object of the generated kernels (empty if none)
  // What it was compiled from, for the second form below: the serialised batch, this routine's
  // position in it, and the options as the caller gave them.
  std::shared_ptr<const std::string> wire;
  int wire_index = 0;
  PlanOptions requested;
  // The same routine planned without any kernel that reads or writes 16 bytes at a time relative to a
  // node's base (matrix-core contractions, row-tile prologues and epilogues): built by the first link
  // that finds one of those operands at a pool offset that is not 16-byte aligned.  The shared layer
  // packs nodes at offsets aligned to the element size only (arrayjit/lib/backends.ml:22-51) and the
  // reference's backends link whatever it hands them (cuda_backend.ml:983-1051).
  mutable std::shared_ptr<CompiledRoutine> unaligned;
};

std::mutex g_mu;
bool g_inited = false;
// process-wide counters behind ocannl_hip_get_global_debug_info
std::atomic<int64_t> g_live_codes{0}, g_compiled_routines{0}, g_hiprtc_modules{0}, g_unaligned_forms{0}, g_routine_runs{0};
std::vector<std::unique_ptr<ocannl_hip_device>> g_devices;

std::vector<char> hiprtc_compile(const std::string& src, const std::string& name) {
  hiprtcProgram prog;
  if (hiprtcCreateProgram(&prog, src.c_str(), (name + ".hip").c_str(), 0, nullptr, nullptr) != HIPRTC_SUCCESS)
    throw RuntimeError("hiprtcCreateProgram failed");
  // No packed-FP32 instructions: they are generated from ordinary float code at -O3 otherwise.
  const char* opts[] = {"--offload-arch=gfx950", "-O3", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                        "-ffp-contract=off"};
  hiprtcResult rc = hiprtcCompileProgram(prog, (int)(sizeof opts / sizeof *opts), opts);
  if (rc != HIPRTC_SUCCESS) {
    size_t n = 0;
    hiprtcGetProgramLogSize(prog, &n);
    std::string log(n, '\0');
    if (n) hiprtcGetProgramLog(prog, &log[0]);
    hiprtcDestroyProgram(&prog);
    // mirrors Cc_backend's "generated code failed to compile" (arrayjit/lib/cc_backend.ml:105-117)
    throw InvalidArgument("hip backend: generated code for " + name + " failed to compile (" +
                          hiprtcGetErrorString(rc) + ")\n" + log);
  }
  size_t n = 0;
  hiprtcGetCodeSize(prog, &n);
  std::vector<char> bin(n);
  hiprtcGetCode(prog, bin.data());
  hiprtcDestroyProgram(&prog);
  ++g_hiprtc_modules;
  return bin;
}

PlanOptions parse_options(const char* options) {
  PlanOptions o;
  if (!options) return o;
  std::stringstream ss(options);
  std::string kv;
  while (std::getline(ss, kv, ';')) {
    if (kv.empty()) continue;
    auto eq = kv.find('=');
    if (eq == std::string::npos) throw InvalidArgument("compile options: expected key=value, got '" + kv + "'");
    const std::string k = kv.substr(0, eq), v = kv.substr(eq + 1);
    if (k == "mfma") o.enable_mfma = v != "0";
    else if (k == "coop") o.enable_coop = v != "0";
    else if (k == "rows") o.enable_row_groups = v != "0";
    else if (k == "bf16_copies") o.enable_bf16_copies = v != "0";
    else if (k == "serial") o.enable_serial_group = v != "0";
    else if (k == "large_models") o.large_models = v != "0";
    else if (k == "groups") o.group_contractions = v != "0";
    else if (k == "chains") o.merge_chains = v != "0";
    else if (k == "side_queue") { o.side_queue = v != "0"; o.side_queue_generated = v == "2"; }
    else if (k == "debug_log") o.debug_log = v != "0";
    else if (k == "row_vec") o.row_vec4 = v != "0";
    else if (k == "graphs") o.use_graphs = v != "0";
    else if (k == "group_window") o.group_window = std::stoi(v);
    else if (k == "epilogues") o.fuse_epilogues = v != "0";
    else if (k == "proj") o.fuse_row_projections = v != "0";
    else if (k == "row_waves") o.row_tile_waves = std::atoi(v.c_str());
    else if (k == "fused") { o.fuse_row_contractions = v != "0"; o.fuse_stored_rows = v == "2"; }
    else if (k == "parallel") o.enable_parallel_groups = v != "0";
    else if (k == "reuse") o.reuse_stored = v != "0";
    else if (k == "min_mfma_flops") o.min_mfma_flops = std::stoll(v);
    else throw InvalidArgument("compile options: unknown key '" + k + "'");
  }
  return o;
}

// Plan, generate and compile cr.r (which the planner rewrites in place).
void build_routine(CompiledRoutine& cr, const PlanOptions& opt) {
  ++g_compiled_routines;
  cr.plan = make_plan(cr.r, opt);
  cr.mod = generate_module(cr.r, cr.plan);
  if (!cr.mod.kernels.empty()) cr.binary = hiprtc_compile(cr.mod.source, cr.r.name);
}

// Nodes whose base address the plan's kernels access 16 bytes at a time.
std::vector<int> wide_access_nodes(const Plan& plan) {
  std::vector<int> ids;
  auto add = [&](int node) { if (node >= 0) ids.push_back(node); };
  for (auto& ph : plan.phases) {
    if (ph.kind == Phase::Contraction) {
      const GemmDesc& g = ph.gemm;
      add(g.a.node); add(g.b.node); add(g.c.node); add(g.c_copy); add(g.epi_bias); add(g.epi_relu);
      for (auto& m : g.group) { add(m.a.node); add(m.b.node); add(m.c.node); add(m.c_copy); }
      for (auto& pr : g.more) { add(pr.first.node); add(pr.second.node); }
    } else if (ph.kind == Phase::Generic) {
      if (ph.fused_x >= 0) { add(ph.fused_a.node); add(ph.fused_b.node); if (ph.fused_x_store) add(ph.fused_x); }
      if (ph.proj_y >= 0) { add(ph.proj_b.node); add(ph.proj_c.node); add(ph.proj_c_copy); }
    }
  }
  return ids;
}

// The form of `cr` that makes no 16-byte access (built once, kept with the code).
const CompiledRoutine& unaligned_form(const CompiledRoutine& cr) {
  static std::mutex mu;
  std::lock_guard<std::mutex> lock(mu);
  if (!cr.unaligned) {
    auto alt = std::make_shared<CompiledRoutine>();
    std::vector<Routine> rs = parse_routines(cr.wire->data(), cr.wire->size());
    alt->r = std::move(rs.at(cr.wire_index));
    alt->wire = cr.wire;
    alt->wire_index = cr.wire_index;
    alt->requested = cr.requested;
    PlanOptions opt = cr.requested;
    opt.enable_mfma = false;
    opt.fuse_row_contractions = opt.fuse_row_projections = opt.fuse_stored_rows = opt.fuse_epilogues = false;
    opt.row_vec4 = false;
    build_routine(*alt, opt);
    ++g_unaligned_forms;
    if (!wide_access_nodes(alt->plan).empty()) throw InvalidArgument("link: the plan without 16-byte accesses still has some");
    cr.unaligned = std::move(alt);
  }
  return *cr.unaligned;
}

}  // namespace

// The compiled routines are shared between the caller's handle and every routine linked from it:
// ocannl_hip_code_free only drops the caller's reference (context_lifetime, cuda_backend.ml:1046-1051).
struct ocannl_hip_code {
  std::shared_ptr<std::vector<CompiledRoutine>> routines = std::make_shared<std::vector<CompiledRoutine>>();
};

struct ocannl_hip_routine {
  ocannl_hip_device* dev = nullptr;
  const CompiledRoutine* code = nullptr;
  std::shared_ptr<std::vector<CompiledRoutine>> keep_code;   // owns what `code` points into
  hipModule_t module = nullptr;
  void* scratch = nullptr;           // the routine's own arena: local nodes, planner scratch, split-K workspace
  uint64_t scratch_bytes = 0;
  bool counted = false;              // included in the device's live_routines
  // Replay: the kernel list of a plain run, captured once per combination of static-index values into
  // a HIP graph (fills recorded as kernels, the side queue as a branch) and launched as one unit from
  // then on: a routine of many short kernels stops paying a host call and a queue round trip per kernel.
  std::map<std::vector<int64_t>, hipGraphExec_t> graphs;
  bool warmed = false;               // one direct run first (it configures kernel attributes)
  int log_id = 0;                    // debug logging: prefix of this run's log lines (cuda_backend.ml:992-993)
  // Everything that names arena memory exists twice: [0] bound to the routine's own arena, [1] bound to
  // the library's static scratch array (valid when static_ok).
  bool static_ok = false;
  void* gemm_ws[2] = {nullptr, nullptr};   // split-K workspace
  void* gemm_ws_side = nullptr;            // ... of the contractions on the side queue (own arena only)
  // side queue: per side-queue phase an event the side queue waits for (recorded on the main queue at
  // the phase's position) and one recorded when the phase has finished; created at link time
  std::map<int, std::pair<hipEvent_t, hipEvent_t>> side_events;
  std::map<int, void*> node_ptr[2];
  std::map<int, int64_t> statics;    // symbol -> current value
  struct Launch {
    int phase = 0;
    hipFunction_t fn = nullptr;
    std::vector<void*> ptr_vals[2];    // storage for pointer arguments
    std::vector<uint64_t> idx_vals;    // storage for static-index arguments (a 32-bit parameter reads the low half)
    std::vector<int> idx_syms;
    int merge_slot = -1;               // index in ptr_vals of the merge-buffer argument, bound at launch
    std::vector<void*> args[2];
    unsigned grid = 1, grid_y = 1, block = 256;
    void* fill_ptr[2] = {nullptr, nullptr}; uint64_t fill_bytes = 0;
  };
  std::vector<Launch> launches;
  std::vector<hipEvent_t> timing_events;
  std::vector<char> profile_mask;           // kernels bracketed with events in plain runs
  std::vector<hipEvent_t> profile_events;   // pairs (start, stop), reused after each read
  size_t profile_used = 0;
};

namespace {

template <class F>
int guarded(F&& f) {
  try {
    f();
    return OCANNL_HIP_OK;
  } catch (const UserError& e) { g_last_error = e.what(); return OCANNL_HIP_E_USER;
  } catch (const InvalidArgument& e) { g_last_error = e.what(); return OCANNL_HIP_E_INVALID;
  } catch (const std::exception& e) { g_last_error = e.what(); return OCANNL_HIP_E_RUNTIME; }
}

void copy_out(const std::string& s, char* buf, size_t cap) {
  if (!buf || cap == 0) throw InvalidArgument("output buffer is null");
  const size_t n = std::min(s.size(), cap - 1);
  std::memcpy(buf, s.data(), n);
  buf[n] = '\0';
}

void destroy_routine(ocannl_hip_routine* rt) {
  if (!rt) return;
  (void)hipSetDevice(rt->dev->ordinal);
  (void)hipStreamSynchronize(rt->dev->stream);
  for (auto e : rt->timing_events) (void)hipEventDestroy(e);
  for (auto& kv : rt->side_events) {
    if (kv.second.first) (void)hipEventDestroy(kv.second.first);
    if (kv.second.second) (void)hipEventDestroy(kv.second.second);
  }
  if (!rt->side_events.empty()) (void)hipStreamSynchronize(rt->dev->side_stream);
  for (auto& kv : rt->graphs) (void)hipGraphExecDestroy(kv.second);
  for (auto e : rt->profile_events) (void)hipEventDestroy(e);
  if (rt->module) (void)hipModuleUnload(rt->module);
  if (rt->scratch) { (void)hipFree(rt->scratch); rt->dev->scratch_used -= rt->scratch_bytes; }
  if (rt->counted) rt->dev->live_routines--;
  delete rt;
}

// `v` = 0: the routine's own arena; 1: the library's static scratch array, with fills as kernels
// and no call that allocates (no events: kernel_ms must be null and bracketing is off).
void enqueue(ocannl_hip_routine& rt, float* kernel_ms, int cap, int v = 0, bool capturing = false) {
  ocannl_hip_device& dev = *rt.dev;
  dev.make_current();
  const Routine& r = rt.code->r;
  // static indices: range check, then publish (cuda_backend.ml:1015-1030)
  for (auto& s : r.statics) {
    const int64_t v = rt.statics[s.sym];
    if (v < 0)
      throw UserError("hip backend: static index " + sym_ident(s.sym) + " is negative: " + std::to_string(v));
    if (s.range >= 0 && v >= s.range)
      throw UserError("hip backend: static index " + sym_ident(s.sym) + " is too big: " + std::to_string(v) +
                      " (range 0.." + std::to_string(s.range - 1) + ")");
    // generated kernels take 32-bit static indices unless the routine was planned with 64-bit offsets
    if (!rt.code->plan.large_index && v > (int64_t)0xFFFFFFFFll)
      throw UserError("hip backend: static index " + sym_ident(s.sym) + " = " + std::to_string(v) +
                      " needs 64-bit indices: compile with large_models=1");
  }
  // the merge buffer is bound when the routine is scheduled, not when it is linked: it may have been
  // regrown since (cuda_backend.ml:1009-1011, :130-134)
  void* merge_base = nullptr;
  if (r.merge_node >= 0) {
    auto it = dev.pools.find(0);
    const uint64_t need = (uint64_t)r.node(r.merge_node).size_in_bytes();
    if (it == dev.pools.end() || it->second.second < need)
      throw UserError("hip backend: routine " + r.name + " reads the merge buffer as " + r.node(r.merge_node).ident +
                      " but no transfer has filled it (device_to_device ~into_merge_buffer first)");
    merge_base = it->second.first;
  }
  if (rt.code->plan.debug_log) {
    static int g_run_id = 0;   // get_global_run_id
    rt.log_id = ++g_run_id;
    // "Debug initial parameter state" (c_syntax.ml:1112-1150): one line per kernel parameter of the
    // routine -- the reference's single kernel prints them itself; here the routine is many kernels, so
    // the host prints them, under the run's log id and ahead of what the kernels print.  Parameters are
    // sorted by their declaration, as c_syntax.ml:1080-1084 sorts them.
    std::vector<std::pair<std::string, std::string>> lines;   // (declaration, rest of the line)
    char buf[64];
    if (r.merge_node >= 0) {
      const Node& n = r.node(r.merge_node);
      snprintf(buf, sizeof buf, "%p", merge_base);
      lines.emplace_back(std::string("const ") + c_typ_name(n.prec) + " *merge_buffer", " &[" + std::to_string(n.num_elems()) + "] = " + buf);
    }
    for (auto& st : r.statics)
      lines.emplace_back(std::string(rt.code->plan.large_index ? "const uint64_t " : "const uint32_t ") + sym_ident(st.sym),
                         " = " + std::to_string(rt.statics.at(st.sym)));
    for (int id : r.node_order) {
      const Node& n = r.node(id);
      if (n.mode != Mode::Ctx) continue;
      snprintf(buf, sizeof buf, "%p", rt.node_ptr[v].at(id));
      lines.emplace_back(std::string(c_typ_name(n.prec)) + " *" + n.ident, " &[" + std::to_string(n.num_elems()) + "] = " + buf);
    }
    std::sort(lines.begin(), lines.end());
    for (auto& l : lines) printf("%d: %s%s$", rt.log_id, l.first.c_str(), l.second.c_str());
    fflush(stdout);
  }
  const bool timed = kernel_ms != nullptr;
  if (timed) {
    if (cap < (int)rt.launches.size()) throw InvalidArgument("run_timed: kernel_ms too small");
    while (rt.timing_events.size() < rt.launches.size() + 1) {
      hipEvent_t e;
      hip_check(hipEventCreate(&e), "hipEventCreate");
      rt.timing_events.push_back(e);
    }
    hip_check(hipEventRecord(rt.timing_events[0], dev.stream), "hipEventRecord");
  }
  // The side queue is used by plain runs over the routine's own arena; per-kernel timing and the
  // static-scratch variant keep everything in order on the main queue.
  const bool two_queues = v == 0 && !timed && !rt.side_events.empty();
  int joined = -1, last_side = -1;   // latest side-queue phase the main queue has waited for / that was launched
  for (size_t li = 0; li < rt.launches.size(); ++li) {
    auto& l = rt.launches[li];
    const Phase& ph = rt.code->plan.phases[l.phase];
    const bool on_side = two_queues && ph.stream == 1;
    hipStream_t stream = on_side ? dev.side_stream : dev.stream;
    if (on_side) {
      auto& ev = rt.side_events.at((int)li);
      hip_check(hipEventRecord(ev.first, dev.stream), "hipEventRecord");
      hip_check(hipStreamWaitEvent(dev.side_stream, ev.first, 0), "hipStreamWaitEvent");
    } else if (two_queues) {
      int need = -1;
      for (int p : ph.wait_for) need = std::max(need, p);
      if (need > joined) {   // (the side queue runs in order: its latest phase stands for the earlier ones)
        hip_check(hipStreamWaitEvent(dev.stream, rt.side_events.at(need).second, 0), "hipStreamWaitEvent");
        joined = need;
      }
    }
    const bool bracket = v == 0 && !timed && li < rt.profile_mask.size() && rt.profile_mask[li];
    if (bracket) {
      while (rt.profile_events.size() < rt.profile_used + 2) {
        hipEvent_t e;
        hip_check(hipEventCreate(&e), "hipEventCreate");
        rt.profile_events.push_back(e);
      }
      hip_check(hipEventRecord(rt.profile_events[rt.profile_used], stream), "hipEventRecord");
    }
    if (ph.kind == Phase::Fill) {
      if (v == 0 && !capturing) {
        hip_check(hipMemsetAsync(l.fill_ptr[0], 0, l.fill_bytes, dev.stream), "hipMemsetAsync");
      } else {
        const uint64_t n16 = l.fill_bytes / 16 + 1;   // one thread per 16-byte store; the first block's 256 threads also cover the <= 15 head and tail bytes
        hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((n16 + 255) / 256)), dim3(256), 0, dev.stream,
                           static_cast<unsigned char*>(l.fill_ptr[v]), l.fill_bytes);
        hip_check(hipGetLastError(), "fill_zero_kernel");
      }
    } else if (ph.kind == Phase::Generic) {
      for (size_t i = 0; i < l.idx_syms.size(); ++i) l.idx_vals[i] = (uint64_t)rt.statics[l.idx_syms[i]];
      if (l.merge_slot >= 0) l.ptr_vals[v][l.merge_slot] = merge_base;
      hip_check(hipModuleLaunchKernel(l.fn, l.grid, l.grid_y, 1, l.block, 1, 1, 0, stream, l.args[v].data(), nullptr),
                "hipModuleLaunchKernel");
    } else {
      const GemmDesc& g = ph.gemm;
      auto base = [&](const GemmOperand& o) -> char* {
        int64_t off = o.offset;
        for (auto& t : o.static_terms) off += rt.statics[t.first] * t.second;
        return static_cast<char*>(rt.node_ptr[v].at(o.node)) + off * prec_in_bytes(o.prec);
      };
      GemmArgs a{};
      a.a = base(g.a); a.b = base(g.b); a.c = base(g.c);
      a.M = g.M; a.N = g.N; a.K = g.K;
      a.a_row = g.a.s_row; a.a_k = g.a.s_k; a.b_row = g.b.s_row; a.b_k = g.b.s_k; a.c_row = g.c.s_row;
      a.nbatch = g.nbatch;
      for (int i = 0; i < 3; ++i) {
        a.batch_ext[i] = g.batch_ext[i];
        a.a_batch[i] = g.a.s_batch[i]; a.b_batch[i] = g.b.s_batch[i]; a.c_batch[i] = g.c.s_batch[i];
      }
      a.accumulate = g.accumulate ? 1 : 0;
      a.c_is_bf16 = g.c.prec == Prec::Bfloat16;
      a.c2 = g.c_copy >= 0 ? rt.node_ptr[v].at(g.c_copy) : nullptr;
      a.bias = g.epi_bias >= 0 ? rt.node_ptr[v].at(g.epi_bias) : nullptr;
      a.relu_out = g.epi_relu >= 0 && g.epi_relu != g.c.node ? rt.node_ptr[v].at(g.epi_relu) : nullptr;
      a.relu_c = g.epi_relu >= 0 && g.epi_relu == g.c.node ? 1 : 0;
      a.npairs = 1 + (int)g.more.size();
      for (size_t p = 0; p < g.more.size(); ++p) { a.a_more[p] = base(g.more[p].first); a.b_more[p] = base(g.more[p].second); }
      a.ngroups = 1 + (int)g.group.size();
      for (size_t m = 0; m < g.group.size(); ++m) {
        a.a_more[m] = base(g.group[m].a); a.b_more[m] = base(g.group[m].b); a.c_more[m] = base(g.group[m].c);
        a.c2_more[m] = g.group[m].c_copy >= 0 ? rt.node_ptr[v].at(g.group[m].c_copy) : nullptr;
      }
      // a bracketed contraction is timed without its split-K reduction (a kernel of its own)
      hip_check(launch_gemm(g, a, on_side ? rt.gemm_ws_side : rt.gemm_ws[v], stream, bracket ? rt.profile_events[rt.profile_used + 1] : nullptr),
                "launch_gemm");
    }
    if (on_side) {
      hip_check(hipEventRecord(rt.side_events.at((int)li).second, dev.side_stream), "hipEventRecord");
      last_side = (int)li;
    }
    if (timed) hip_check(hipEventRecord(rt.timing_events[li + 1], dev.stream), "hipEventRecord");
    if (bracket) {
      if (ph.kind != Phase::Contraction)
        hip_check(hipEventRecord(rt.profile_events[rt.profile_used + 1], stream), "hipEventRecord");
      rt.profile_used += 2;
    }
  }
  // whatever follows on the main queue (the caller's copies, the next run) comes after the side queue's work
  if (last_side > joined) hip_check(hipStreamWaitEvent(dev.stream, rt.side_events.at(last_side).second, 0), "hipStreamWaitEvent");
  if (timed) {
    hip_check(hipStreamSynchronize(dev.stream), "hipStreamSynchronize");
    for (size_t li = 0; li < rt.launches.size(); ++li)
      hip_check(hipEventElapsedTime(&kernel_ms[li], rt.timing_events[li], rt.timing_events[li + 1]), "hipEventElapsedTime");
  }
}

}  // namespace

// ================================================================================================
extern "C" {

const char* ocannl_hip_last_error(void) { return g_last_error.c_str(); }

int ocannl_hip_init(void) {
  return guarded([] {
    std::lock_guard<std::mutex> lk(g_mu);
    if (g_inited) return;
    hip_check(hipInit(0), "hipInit");
    int n = 0;
    hip_check(hipGetDeviceCount(&n), "hipGetDeviceCount");
    g_devices.resize(n);
    g_inited = true;
  });
}

int ocannl_hip_num_devices(int* count) {
  return guarded([&] {
    if (!count) throw InvalidArgument("num_devices: null output");
    if (!g_inited) { int rc = ocannl_hip_init(); if (rc) throw RuntimeError(g_last_error); }
    *count = (int)g_devices.size();
  });
}

int ocannl_hip_get_device(int ordinal, ocannl_hip_device** out) {
  return guarded([&] {
    if (!out) throw InvalidArgument("get_device: null output");
    if (!g_inited) { int rc = ocannl_hip_init(); if (rc) throw RuntimeError(g_last_error); }
    std::lock_guard<std::mutex> lk(g_mu);
    if (ordinal < 0 || ordinal >= (int)g_devices.size())
      throw InvalidArgument("get_device: ordinal " + std::to_string(ordinal) + " out of range (" +
                            std::to_string(g_devices.size()) + " devices)");
    if (!g_devices[ordinal]) {
      auto d = std::make_unique<ocannl_hip_device>();
      d->ordinal = ordinal;
      d->make_current();
      hip_check(hipGetDeviceProperties(&d->props, ordinal), "hipGetDeviceProperties");
      if (std::string(d->props.gcnArchName).rfind("gfx950", 0) != 0)
        throw RuntimeError(std::string("hip backend: device is ") + d->props.gcnArchName + ", this library is built for gfx950 only");
      hip_check(hipStreamCreateWithFlags(&d->stream, hipStreamNonBlocking), "hipStreamCreateWithFlags");
      hip_check(hipStreamCreateWithFlags(&d->side_stream, hipStreamNonBlocking), "hipStreamCreateWithFlags");
      // this device's address of the library's static scratch array (the device is current here)
      hip_check(hipGetSymbolAddress(&d->static_scratch, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)");
      g_devices[ordinal] = std::move(d);
    }
    *out = g_devices[ordinal].get();
  });
}

int ocannl_hip_get_name(ocannl_hip_device* dev, char* buf, size_t cap) {
  return guarded([&] {
    if (!dev) throw InvalidArgument("get_name: null device");
    copy_out("hip:" + std::to_string(dev->ordinal), buf, cap);
  });
}

int ocannl_hip_static_properties(char* buf, size_t cap) {
  return guarded([&] {
    if (!g_inited) { int rc = ocannl_hip_init(); if (rc) throw RuntimeError(g_last_error); }
    std::ostringstream s;
    s << "(";
    for (size_t i = 0; i < g_devices.size(); ++i) {
      hipDeviceProp_t p;
      hip_check(hipGetDeviceProperties(&p, (int)i), "hipGetDeviceProperties");
      s << "((device " << i << ") (name \"" << p.name << "\") (arch " << p.gcnArchName << ") (total_global_mem "
        << p.totalGlobalMem << ") (multiprocessor_count " << p.multiProcessorCount << ") (warp_size " << p.warpSize
        << ") (max_shared_memory_per_block " << p.sharedMemPerBlock << ") (clock_rate_khz " << p.clockRate
        << ") (memory_clock_rate_khz " << p.memoryClockRate << ") (memory_bus_width " << p.memoryBusWidth
        << ") (l2_cache_size " << p.l2CacheSize << "))";
    }
    s << ")";
    copy_out(s.str(), buf, cap);
  });
}

int ocannl_hip_get_used_memory(ocannl_hip_device* dev, uint64_t* bytes) {
  return guarded([&] {
    if (!dev || !bytes) throw InvalidArgument("get_used_memory: null argument");
    *bytes = dev->used + dev->scratch_used;
  });
}

int ocannl_hip_get_debug_info(ocannl_hip_device* dev, char* buf, size_t cap) {
  return guarded([&] {
    if (!dev) throw InvalidArgument("get_debug_info: null device");
    std::ostringstream s;
    s << "((pools " << dev->pools.size() << ") (pool_bytes " << dev->used << ") (scratch_bytes " << dev->scratch_used
      << ") (live_events " << dev->live_events << ") (live_routines " << dev->live_routines << "))";
    copy_out(s.str(), buf, cap);
  });
}

int ocannl_hip_get_global_debug_info(char* buf, size_t cap) {
  return guarded([&] {
    std::lock_guard<std::mutex> lock(g_mu);
    int64_t devices = 0, pools = 0, pool_bytes = 0, scratch_bytes = 0, events = 0, routines = 0;
    for (auto& d : g_devices) {
      if (!d) continue;
      ++devices;
      pools += (int64_t)d->pools.size(); pool_bytes += (int64_t)d->used; scratch_bytes += (int64_t)d->scratch_used;
      events += d->live_events; routines += d->live_routines;
    }
    std::ostringstream s;
    s << "(hip_global_debug (live_devices " << devices << ") (live_streams " << devices << ") (live_events " << events
      << ") (live_codes " << g_live_codes.load() << ") (live_routines " << routines << ") (compiled_routines "
      << g_compiled_routines.load() << ") (hiprtc_modules " << g_hiprtc_modules.load() << ") (unaligned_forms "
      << g_unaligned_forms.load() << ") (routine_runs " << g_routine_runs.load() << ") (pools " << pools << ") (pool_bytes "
      << pool_bytes << ") (scratch_bytes " << scratch_bytes << "))";
    copy_out(s.str(), buf, cap);
  });
}

int ocannl_hip_await(ocannl_hip_device* dev) {
  return guarded([&] {
    if (!dev) throw InvalidArgument("await: null device");
    dev->make_current();
    hip_check(hipStreamSynchronize(dev->stream), "hipStreamSynchronize");
  });
}

int ocannl_hip_is_idle(ocannl_hip_device* dev, int* idle) {
  return guarded([&] {
    if (!dev || !idle) throw InvalidArgument("is_idle: null argument");
    dev->make_current();
    hipError_t e = hipStreamQuery(dev->stream);
    if (e == hipSuccess) *idle = 1;
    else if (e == hipErrorNotReady) *idle = 0;
    else hip_check(e, "hipStreamQuery");
  });
}

int ocannl_hip_all_work(ocannl_hip_device* dev, ocannl_hip_event** out) {
  return guarded([&] {
    if (!dev || !out) throw InvalidArgument("all_work: null argument");
    dev->make_current();
    auto ev = std::make_unique<ocannl_hip_event>();
    ev->dev = dev;
    hip_check(hipEventCreateWithFlags(&ev->ev, hipEventDisableTiming), "hipEventCreateWithFlags");
    hip_check(hipEventRecord(ev->ev, dev->stream), "hipEventRecord");
    dev->live_events++;
    *out = ev.release();
  });
}

int ocannl_hip_sync(ocannl_hip_event* ev) {
  return guarded([&] {
    if (!ev) throw InvalidArgument("sync: null event");
    ev->dev->make_current();
    hip_check(hipEventSynchronize(ev->ev), "hipEventSynchronize");
  });
}

int ocannl_hip_is_done(ocannl_hip_event* ev, int* done) {
  return guarded([&] {
    if (!ev || !done) throw InvalidArgument("is_done: null argument");
    ev->dev->make_current();
    hipError_t e = hipEventQuery(ev->ev);
    if (e == hipSuccess) *done = 1;
    else if (e == hipErrorNotReady) *done = 0;
    else hip_check(e, "hipEventQuery");
  });
}

int ocannl_hip_will_wait_for(ocannl_hip_device* dev, ocannl_hip_event* ev) {
  return guarded([&] {
    if (!dev || !ev) throw InvalidArgument("will_wait_for: null argument");
    dev->make_current();
    hip_check(hipStreamWaitEvent(dev->stream, ev->ev, 0), "hipStreamWaitEvent");
  });
}

void ocannl_hip_event_free(ocannl_hip_event* ev) {
  if (!ev) return;
  if (ev->ev) (void)hipEventDestroy(ev->ev);
  ev->dev->live_events--;
  delete ev;
}

int ocannl_hip_alloc_pool(ocannl_hip_device* dev, int pool_id, uint64_t size, uint64_t alignment) {
  return guarded([&] {
    if (!dev) throw InvalidArgument("alloc_pool: null device");
    if (alignment > 256) throw InvalidArgument("alloc_pool: alignment above 256 bytes is not supported");
    dev->make_current();
    auto it = dev->pools.find(pool_id);
    if (it != dev->pools.end()) {   // regrowth: release the old slab first
      hip_check(hipStreamSynchronize(dev->stream), "hipStreamSynchronize");
      hip_check(hipFree(it->second.first), "hipFree");
      dev->used -= it->second.second;
      dev->pools.erase(it);
    }
    void* p = nullptr;
    hip_check(hipMalloc(&p, size ? size : 1), "hipMalloc");
    dev->pools[pool_id] = {p, size};
    dev->used += size;
  });
}

int ocannl_hip_free_pool(ocannl_hip_device* dev, int pool_id) {
  return guarded([&] {
    if (!dev) throw InvalidArgument("free_pool: null device");
    auto it = dev->pools.find(pool_id);
    if (it == dev->pools.end()) throw InvalidArgument("free_pool: unknown pool_id " + std::to_string(pool_id));
    dev->make_current();
    hip_check(hipStreamSynchronize(dev->stream), "hipStreamSynchronize");
    hip_check(hipFree(it->second.first), "hipFree");
    dev->used -= it->second.second;
    dev->pools.erase(it);
  });
}

int ocannl_hip_memset_zero(ocannl_hip_device* dev, int pool_id, uint64_t offset, uint64_t size) {
  return guarded([&] {
    if (!dev) throw InvalidArgument("memset_zero: null device");
    dev->make_current();
    void* p = dev->resolve(pool_id, offset, size, "memset_zero");
    if (size) hip_check(hipMemsetAsync(p, 0, size, dev->stream), "hipMemsetAsync");
  });
}

int ocannl_hip_from_host(ocannl_hip_device* dev, int pool_id, uint64_t offset, const void* src, uint64_t bytes) {
  return guarded([&] {
    if (!dev || (!src && bytes)) throw InvalidArgument("from_host: null argument");
    dev->make_current();
    void* p = dev->resolve(pool_id, offset, bytes, "from_host");
    if (bytes) hip_check(hipMemcpyAsync(p, src, bytes, hipMemcpyHostToDevice, dev->stream), "hipMemcpyAsync(H2D)");
  });
}

int ocannl_hip_to_host(ocannl_hip_device* dev, int pool_id, uint64_t offset, void* dst, uint64_t bytes) {
  return guarded([&] {
    if (!dev || (!dst && bytes)) throw InvalidArgument("to_host: null argument");
    dev->make_current();
    void* p = dev->resolve(pool_id, offset, bytes, "to_host");
    if (bytes) hip_check(hipMemcpyAsync(dst, p, bytes, hipMemcpyDeviceToHost, dev->stream), "hipMemcpyAsync(D2H)");
  });
}

int ocannl_hip_device_to_device(ocannl_hip_device* dst, int dst_pool, uint64_t dst_off, ocannl_hip_device* src,
                                int src_pool, uint64_t src_off, uint64_t bytes) {
  return guarded([&] {
    if (!dst || !src) throw InvalidArgument("device_to_device: null device");
    if (dst_pool < 0) {   // into the merge buffer = pool 0, grown on demand
      auto it = dst->pools.find(0);
      if (it == dst->pools.end() || it->second.second < bytes) {
        int rc = ocannl_hip_alloc_pool(dst, 0, bytes, 256);
        if (rc) throw RuntimeError(g_last_error);
      }
      dst_pool = 0; dst_off = 0;
    }
    void* d = dst->resolve(dst_pool, dst_off, bytes, "device_to_device(dst)");
    void* s = src->resolve(src_pool, src_off, bytes, "device_to_device(src)");
    dst->make_current();
    if (dst->ordinal == src->ordinal) {
      if (d == s) return;
      hip_check(hipMemcpyAsync(d, s, bytes, hipMemcpyDeviceToDevice, dst->stream), "hipMemcpyAsync(D2D)");
    } else {
      hip_check(hipMemcpyPeerAsync(d, dst->ordinal, s, src->ordinal, bytes, dst->stream), "hipMemcpyPeerAsync");
    }
  });
}

int ocannl_hip_compile_opts(const char* llir, size_t len, const char* options, ocannl_hip_code** out) {
  return guarded([&] {
    if (!llir || !out) throw InvalidArgument("compile: null argument");
    PlanOptions opt = parse_options(options);
    auto code = std::make_unique<ocannl_hip_code>();
    auto wire = std::make_shared<const std::string>(llir, len);
    std::vector<Routine> rs = parse_routines(llir, len);
    for (auto& r : rs) {
      CompiledRoutine cr;
      cr.r = std::move(r);
      cr.wire = wire;
      cr.wire_index = (int)code->routines->size();
      cr.requested = opt;
      build_routine(cr, opt);
      code->routines->push_back(std::move(cr));
    }
    *out = code.release();
    ++g_live_codes;
  });
}

int ocannl_hip_compile(const char* llir, size_t len, ocannl_hip_code** out) {
  return ocannl_hip_compile_opts(llir, len, nullptr, out);
}

void ocannl_hip_code_free(ocannl_hip_code* code) {
  if (code) --g_live_codes;
  delete code;
}

static const CompiledRoutine& routine_at(ocannl_hip_code* code, int index) {
  if (!code) throw InvalidArgument("null code");
  if (index < 0 || index >= (int)code->routines->size()) throw InvalidArgument("routine index out of range");
  return (*code->routines)[index];
}

int ocannl_hip_code_num_routines(ocannl_hip_code* code, int* n) {
  return guarded([&] { if (!code || !n) throw InvalidArgument("null argument"); *n = (int)code->routines->size(); });
}

int ocannl_hip_code_routine_name(ocannl_hip_code* code, int index, char* buf, size_t cap) {
  return guarded([&] { copy_out(routine_at(code, index).r.name, buf, cap); });
}

int ocannl_hip_code_kparams(ocannl_hip_code* code, int index, ocannl_hip_kparam* params, int cap, int* count) {
  return guarded([&] {
    const CompiledRoutine& cr = routine_at(code, index);
    std::vector<ocannl_hip_kparam> ks;
    if (cr.r.merge_node >= 0) ks.push_back({2, cr.r.merge_node, cr.r.node(cr.r.merge_node).size_in_bytes()});
    for (auto& s : cr.r.statics) ks.push_back({1, s.sym, s.range});
    for (int id : cr.r.node_order) {
      const Node& n = cr.r.node(id);
      if (n.mode == Mode::Ctx) ks.push_back({0, id, n.size_in_bytes()});
    }
    if (count) *count = (int)ks.size();
    if (params) {
      if (cap < (int)ks.size()) throw InvalidArgument("kparams: buffer too small");
      std::copy(ks.begin(), ks.end(), params);
    }
  });
}

int ocannl_hip_code_source(ocannl_hip_code* code, char* buf, size_t cap, size_t* needed) {
  return guarded([&] {
    if (!code) throw InvalidArgument("null code");
    std::string all;
    for (auto& cr : *code->routines) all += cr.mod.source;
    if (needed) *needed = all.size() + 1;
    if (buf) copy_out(all, buf, cap);
  });
}

int ocannl_hip_code_object(ocannl_hip_code* code, int index, char* buf, size_t cap, size_t* needed) {
  return guarded([&] {
    const CompiledRoutine& cr = routine_at(code, index);
    if (needed) *needed = cr.binary.size();
    if (buf) {
      if (cap < cr.binary.size()) throw InvalidArgument("code_object: buffer too small");
      std::memcpy(buf, cr.binary.data(), cr.binary.size());
    }
  });
}

int ocannl_hip_code_num_kernels(ocannl_hip_code* code, int index, int* n) {
  return guarded([&] { if (!n) throw InvalidArgument("null argument"); *n = (int)routine_at(code, index).plan.phases.size(); });
}

int ocannl_hip_code_kernel_info(ocannl_hip_code* code, int index, int kernel, ocannl_hip_kernel_info* info) {
  return guarded([&] {
    const CompiledRoutine& cr = routine_at(code, index);
    if (!info || kernel < 0 || kernel >= (int)cr.plan.phases.size()) throw InvalidArgument("kernel index out of range");
    const Phase& ph = cr.plan.phases[kernel];
    std::memset(info, 0, sizeof *info);
    info->kind = ph.kind == Phase::Generic ? 0 : ph.kind == Phase::Fill ? 1 : 2;
    info->coop_lanes = ph.coop_lanes;
    info->flops = ph.flops;
    info->bytes = ph.bytes;
    info->queue = ph.stream;
    std::string name;
    if (ph.kind == Phase::Contraction) {
      // grouped contractions read as more batch entries, a chain of operand pairs as a longer K
      info->m = ph.gemm.M; info->n = ph.gemm.N; info->k = ph.gemm.K * (int64_t)(1 + ph.gemm.more.size());
      info->batch = 1 + (int64_t)ph.gemm.group.size();
      for (int i = 0; i < ph.gemm.nbatch; ++i) info->batch *= ph.gemm.batch_ext[i];
      name = gemm_kernel_name(ph.gemm);
    } else if (ph.kind == Phase::Fill) {
      name = "fill_zero:" + cr.r.node(ph.fill_node).ident;
    } else {
      for (auto& k : cr.mod.kernels) if (k.phase_index == kernel) name = k.name;
    }
    copy_out(name, info->name, sizeof info->name);
  });
}

int ocannl_hip_link(ocannl_hip_device* dev, ocannl_hip_code* code, int index, const ocannl_hip_node_loc* locs, int n_locs,
                    ocannl_hip_routine** out) {
  return guarded([&] {
    if (!dev || !out) throw InvalidArgument("link: null argument");
    const CompiledRoutine& requested = routine_at(code, index);
    if (n_locs > 0 && !locs) throw InvalidArgument("link: null locs");
    dev->make_current();
    // The matrix-core kernels and the row-tile prologues / epilogues read and write 16-byte chunks
    // relative to a node's base (local nodes sit at 256-byte offsets).  A context node that one of
    // them touches at a pool offset that is not 16-byte aligned selects the routine's other form,
    // in which generated kernels do that work element by element.
    bool misaligned = false;
    {
      std::map<int, const ocannl_hip_node_loc*> where;
      for (int i = 0; i < n_locs; ++i) where[locs[i].node_id] = &locs[i];
      for (int id : wide_access_nodes(requested.plan)) {
        auto it = where.find(id);
        if (it == where.end() || requested.r.node(id).mode != Mode::Ctx) continue;
        auto pool = dev->pools.find(it->second->pool_id);
        const uintptr_t base = pool == dev->pools.end() ? 0 : reinterpret_cast<uintptr_t>(pool->second.first);
        if ((base + it->second->offset) % 16 != 0) misaligned = true;
      }
    }
    const CompiledRoutine& cr = misaligned ? unaligned_form(requested) : requested;
    // anything that fails below releases what the routine holds so far
    std::unique_ptr<ocannl_hip_routine, void (*)(ocannl_hip_routine*)> rt(new ocannl_hip_routine, destroy_routine);
    rt->dev = dev;
    rt->code = &cr;
    rt->keep_code = code->routines;
    // ctx nodes from the caller's table: checked before anything is allocated
    std::map<int, const ocannl_hip_node_loc*> by_id;
    for (int i = 0; i < n_locs; ++i) by_id[locs[i].node_id] = &locs[i];
    std::map<int, void*> ctx_ptr;
    for (auto& kv : cr.r.nodes) {
      const Node& n = kv.second;
      if (n.mode != Mode::Ctx) continue;
      auto it = by_id.find(n.id);
      if (it == by_id.end())
        throw UserError("hip backend link: node " + n.ident + " (id " + std::to_string(n.id) + ") missing from context");
      ctx_ptr[n.id] = dev->resolve(it->second->pool_id, it->second->offset, (uint64_t)n.size_in_bytes(), "link");
    }
    // local nodes (and planner scratch): one private arena, 256-byte aligned sub-buffers
    uint64_t arena = 0;
    std::map<int, uint64_t> local_off;
    for (auto& kv : cr.r.nodes) {
      const Node& n = kv.second;
      if (n.mode != Mode::Local) continue;
      local_off[n.id] = arena;
      arena += ((uint64_t)n.size_in_bytes() + 255) / 256 * 256;
    }
    uint64_t ws_bytes = 0, ws_side_bytes = 0;
    for (auto& ph : cr.plan.phases)
      if (ph.kind == Phase::Contraction) {
        ws_bytes = std::max<uint64_t>(ws_bytes, gemm_workspace_bytes(ph.gemm));   // (any phase may run on the main queue)
        if (ph.stream == 1) ws_side_bytes = std::max<uint64_t>(ws_side_bytes, gemm_workspace_bytes(ph.gemm));
      }
    const uint64_t ws_off = arena;
    arena += (ws_bytes + 255) / 256 * 256;
    const uint64_t ws_side_off = arena;
    arena += (ws_side_bytes + 255) / 256 * 256;
    rt->scratch_bytes = arena;
    if (arena) {
      hip_check(hipMalloc(&rt->scratch, arena), "hipMalloc(scratch)");
      dev->scratch_used += arena;
    }
    // Two bindings of the same kernel list: [0] over the routine's own arena, [1] over the library's
    // static scratch array (only when the arena fits into it).
    char* const bases[2] = {static_cast<char*>(rt->scratch), static_cast<char*>(dev->static_scratch)};
    rt->static_ok = arena <= kStaticScratchBytes && dev->static_scratch != nullptr;
    for (int v = 0; v < 2; ++v) {
      if (v == 1 && !rt->static_ok) break;
      rt->node_ptr[v] = ctx_ptr;
      for (auto& kv : local_off) rt->node_ptr[v][kv.first] = bases[v] + kv.second;
      rt->gemm_ws[v] = ws_bytes ? bases[v] + ws_off : nullptr;
    }
    rt->gemm_ws_side = ws_side_bytes ? bases[0] + ws_side_off : nullptr;
    for (size_t pi = 0; pi < cr.plan.phases.size(); ++pi) {
      if (cr.plan.phases[pi].stream != 1) continue;
      std::pair<hipEvent_t, hipEvent_t> ev{nullptr, nullptr};
      hip_check(hipEventCreateWithFlags(&ev.first, hipEventDisableTiming), "hipEventCreateWithFlags");
      rt->side_events[(int)pi] = ev;   // (registered before the second is made, so that a failure releases the first)
      hip_check(hipEventCreateWithFlags(&rt->side_events[(int)pi].second, hipEventDisableTiming), "hipEventCreateWithFlags");
    }
    for (auto& s : cr.r.statics) rt->statics[s.sym] = 0;
    if (!cr.binary.empty()) hip_check(hipModuleLoadData(&rt->module, cr.binary.data()), "hipModuleLoadData");
    // launch records
    size_t next_generic = 0;
    rt->launches.resize(cr.plan.phases.size());
    for (size_t pi = 0; pi < cr.plan.phases.size(); ++pi) {
      const Phase& ph = cr.plan.phases[pi];
      ocannl_hip_routine::Launch& l = rt->launches[pi];
      l.phase = (int)pi;
      if (ph.kind == Phase::Fill) {
        for (int v = 0; v < (rt->static_ok ? 2 : 1); ++v) l.fill_ptr[v] = rt->node_ptr[v].at(ph.fill_node);
        l.fill_bytes = (uint64_t)cr.r.node(ph.fill_node).size_in_bytes();
      } else if (ph.kind == Phase::Generic) {
        const GeneratedKernel& gk = cr.mod.kernels.at(next_generic++);
        if (gk.phase_index != (int)pi) throw InvalidArgument("link: kernel table out of step with the plan");
        hip_check(hipModuleGetFunction(&l.fn, rt->module, gk.name.c_str()), "hipModuleGetFunction");
        const uint64_t blocks = (gk.threads + gk.block - 1) / gk.block;
        // a launch may not exceed 2^32 threads along one grid dimension: rows of 2^22 workgroups
        constexpr uint64_t kRow = 1ull << 22;
        if (blocks == 0 || blocks > kRow * 65535ull) throw UserError("hip backend: phase too large for one launch: " + gk.name);
        l.grid = (unsigned)std::min(blocks, kRow);
        l.grid_y = (unsigned)((blocks + kRow - 1) / kRow);
        l.block = (unsigned)gk.block;
        size_t np = 0, ni = 0;
        for (auto& p : gk.params) {
          if (p.kind == KernelParam::StaticIdx) ++ni;
          else if (p.kind != KernelParam::LogId) ++np;
        }
        // (sized once: the argument arrays below point into these vectors)
        l.idx_vals.assign(ni, 0);
        for (auto& p : gk.params) if (p.kind == KernelParam::StaticIdx) l.idx_syms.push_back(p.id);
        for (int v = 0; v < (rt->static_ok ? 2 : 1); ++v) {
          l.ptr_vals[v].assign(np, nullptr);
          size_t ip = 0, ii = 0;
          for (auto& p : gk.params) {
            if (p.kind == KernelParam::StaticIdx) { l.args[v].push_back(&l.idx_vals[ii++]); continue; }
            if (p.kind == KernelParam::LogId) { l.args[v].push_back(&rt->log_id); continue; }
            if (p.kind == KernelParam::NodePtr) l.ptr_vals[v][ip] = rt->node_ptr[v].at(p.id);
            else l.merge_slot = (int)ip;
            l.args[v].push_back(&l.ptr_vals[v][ip++]);
          }
        }
      }
    }
    dev->live_routines++;
    rt->counted = true;
    *out = rt.release();
  });
}

void ocannl_hip_routine_free(ocannl_hip_routine* rt) { destroy_routine(rt); }

int ocannl_hip_routine_set_static(ocannl_hip_routine* rt, int symbol, int64_t value) {
  return guarded([&] {
    if (!rt) throw InvalidArgument("set_static: null routine");
    auto it = rt->statics.find(symbol);
    if (it == rt->statics.end()) throw InvalidArgument("set_static: routine has no static index " + sym_ident(symbol));
    it->second = value;
  });
}

// A plain run, replayed from a captured graph when it can be: several kernels, no merge buffer (bound
// at launch), no event bracketing, no device printing, and a graph for this combination of static indices
// (at most kMaxGraphs of them are kept; beyond that, and on the very first run, the kernels are
// launched one by one).
static void run_plain(ocannl_hip_routine& rt) {
  constexpr size_t kMaxGraphs = 128;
  const auto& plan = rt.code->plan;
  bool bracketing = false;
  for (char m : rt.profile_mask) bracketing = bracketing || m;
  const bool graphable = plan.use_graphs && rt.launches.size() >= 2 && rt.code->r.merge_node < 0 && !bracketing && !plan.debug_log;
  if (!graphable || !rt.warmed) { enqueue(rt, nullptr, 0); rt.warmed = true; return; }
  std::vector<int64_t> key;
  for (auto& s : rt.code->r.statics) key.push_back(rt.statics[s.sym]);
  auto it = rt.graphs.find(key);
  ocannl_hip_device& dev = *rt.dev;
  if (it == rt.graphs.end()) {
    if (rt.graphs.size() >= kMaxGraphs) { enqueue(rt, nullptr, 0); return; }
    dev.make_current();
    hip_check(hipStreamBeginCapture(dev.stream, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture");
    hipGraph_t graph = nullptr;
    try {
      enqueue(rt, nullptr, 0, 0, true);
    } catch (...) {
      (void)hipStreamEndCapture(dev.stream, &graph);
      if (graph) (void)hipGraphDestroy(graph);
      throw;
    }
    hip_check(hipStreamEndCapture(dev.stream, &graph), "hipStreamEndCapture");
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    hip_check(e, "hipGraphInstantiate");
    it = rt.graphs.emplace(key, exec).first;
  }
  dev.make_current();
  hip_check(hipGraphLaunch(it->second, dev.stream), "hipGraphLaunch");
}

int ocannl_hip_routine_run(ocannl_hip_routine* rt) {
  return guarded([&] {
    if (!rt) throw InvalidArgument("run: null routine");
    ++g_routine_runs;
    run_plain(*rt);
  });
}

int ocannl_hip_routine_run_static_scratch(ocannl_hip_routine* rt) {
  return guarded([&] {
    if (!rt) throw InvalidArgument("run_static_scratch: null routine");
    if (rt->scratch_bytes > kStaticScratchBytes)
      throw UserError("hip backend: routine " + rt->code->r.name + " needs " + std::to_string(rt->scratch_bytes) +
                      " bytes of scratch memory, above the " + std::to_string(kStaticScratchBytes) +
                      " bytes of the library's static scratch array: use ocannl_hip_routine_run");
    if (!rt->static_ok) throw RuntimeError("run_static_scratch: the device's static scratch array was not set up");
    enqueue(*rt, nullptr, 0, 1);
  });
}

int ocannl_hip_routine_log_id(ocannl_hip_routine* rt, int* log_id) {
  return guarded([&] {
    if (!rt || !log_id) throw InvalidArgument("log_id: null argument");
    *log_id = rt->log_id;
  });
}

int ocannl_hip_routine_run_timed(ocannl_hip_routine* rt, float* kernel_ms, int cap) {
  return guarded([&] {
    if (!rt || !kernel_ms) throw InvalidArgument("run_timed: null argument");
    enqueue(*rt, kernel_ms, cap);
  });
}

int ocannl_hip_routine_profile_kernel(ocannl_hip_routine* rt, int kernel_index) {
  return guarded([&] {
    if (!rt) throw InvalidArgument("profile_kernel: null routine");
    if (kernel_index >= (int)rt->launches.size()) throw InvalidArgument("profile_kernel: kernel index out of range");
    if (kernel_index < 0) { rt->profile_mask.clear(); return; }
    rt->profile_mask.resize(rt->launches.size(), 0);
    rt->profile_mask[kernel_index] = 1;
  });
}

int ocannl_hip_routine_profile_read(ocannl_hip_routine* rt, double* total_ms, int64_t* launches) {
  return guarded([&] {
    if (!rt || !total_ms || !launches) throw InvalidArgument("profile_read: null argument");
    rt->dev->make_current();
    hip_check(hipStreamSynchronize(rt->dev->stream), "hipStreamSynchronize");
    double sum = 0;
    for (size_t i = 0; i + 1 < rt->profile_used; i += 2) {
      float ms = 0;
      hip_check(hipEventElapsedTime(&ms, rt->profile_events[i], rt->profile_events[i + 1]), "hipEventElapsedTime");
      sum += ms;
    }
    *total_ms = sum;
    *launches = (int64_t)(rt->profile_used / 2);
    rt->profile_used = 0;
  });
}

}  // extern "C"
