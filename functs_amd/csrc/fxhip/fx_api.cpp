// C ABI of libfxhip (see include/fxhip.h) and the launch-time runtime:
// argument marshalling into the by-value FxDyn block, one-time upload of the
// static region blob, kernel launches on the caller's stream.
//
// Counterpart of GraphBuilder::prepareRunArgs / runKernel
// (fait/fuser/graph_builder.cpp:718-927) and CudaCodeGenTssa::call_raw
// (fait/tensorexpr/cuda_codegen_tssa.cpp:1167-1290).
#ifndef FX_DENSE_WG_PER_CU
#define FX_DENSE_WG_PER_CU 12u   // workgroups of the dense kernel per CU (4 are resident; more, smaller shares even out the tail: measured 4 to 16)
#endif
#include <hip/hip_runtime.h>

#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "fx_lower.h"

struct FxSpecKernels;
const FxSpecKernels* fx_spec_find(uint64_t hash);
int fx_spec_count();
hipError_t fx_launch_dense(int rank, const uint32_t* sb, const FxLaunchInfo& li, const FxDyn* dyn, uint32_t grid,
                           hipStream_t stream, const FxSpecKernels* spec, const FxLeanArgs* lean, uint32_t slot_err);
hipError_t fx_launch_compact_count(const uint32_t* sb, const FxLaunchInfo& li, const FxDyn* dyn, uint32_t grid,
                                   hipStream_t stream, const FxSpecKernels* spec);
hipError_t fx_launch_compact_scatter(int rank, const uint32_t* sb, const FxLaunchInfo& li, const FxDyn* dyn,
                                     uint32_t grid, hipStream_t stream, const FxSpecKernels* spec);
hipError_t fx_launch_copy(const void* src, void* dst, size_t bytes, uint32_t grid, hipStream_t stream);
hipError_t fx_launch_compact_stream(int rank, const uint32_t* sb, const FxLaunchInfo& li, const FxDyn* dyn, uint32_t grid,
                                    hipStream_t stream, const FxSpecKernels* spec);
uint32_t fx_stream_lds_bytes(const FxLaunchInfo& li, bool compiled);
bool fx_spec_has_stream(const FxSpecKernels* spec);
bool fx_spec_has_lean(const FxSpecKernels* spec);
// fx_head.hip
hipError_t fx_launch_head_stream(const FxHeadLaunch& hl, const FxDyn* dyn, hipStream_t stream);
hipError_t fx_upload_words(const uint64_t* words, size_t n_words, void* dst, hipStream_t stream);
hipError_t fx_head_resident(uint32_t lds_bytes, uint32_t* workgroups, uint32_t* per_cu);
uint32_t fx_head_lds_bytes(const FxHeadLaunch& hl);
// fx_cmap.hip
hipError_t fx_launch_classmap_head(const FxCmapLaunch& hl, const FxDyn* dyn, bool wide, hipStream_t stream);
hipError_t fx_cmap_resident(uint32_t lds_bytes, uint32_t* wide, uint32_t* narrow);
uint32_t fx_cmap_lds_bytes(const FxCmapLaunch& hl);
uint32_t fx_cmap_chunk_rows();
#include "fx_lstm_sched.h"
int fx_launch_lstm_stack(const FxLstmArgs& a, int L, hipStream_t stream);
int fx_launch_sort_nms(const fx_nms_desc& d, uint32_t key_cap, void* workspace, uint32_t* err_host, hipStream_t stream);
size_t fx_nms_workspace_bytes(int n_tasks, uint32_t key_cap);
size_t fx_nms_workspace_clear_bytes(int n_tasks);
hipError_t fx_launch_compact_rows_static(const uint8_t* mask, int64_t n, const void* const* cols, void* const* outs,
                                         const int32_t* rowlen, const int32_t* elsize, int n_cols,
                                         uint32_t* total_host, hipStream_t stream);
hipError_t fx_launch_compact_rows(const uint8_t* mask, int64_t n, const void* const* cols, void* const* outs,
                                  const int32_t* rowlen, const int32_t* elsize, int n_cols, uint32_t* counts,
                                  uint32_t* total_host, hipStream_t stream);

struct fx_region {
  fx::Region r;
  std::mutex mu;  // plan cache + device upload (the reference serialises extent
                  // evaluation the same way, cuda_codegen_tssa.cpp:1207)
};
struct fx_plan {
  fx::Plan p;
};

namespace {

thread_local std::string g_err;

int fail(int code, const std::string& msg) {
  g_err = msg;
  return code;
}

#define FX_TRY try {
#define FX_CATCH                                                   \
  }                                                                \
  catch (const fx::Error& e) { return fail(e.code, e.what()); }    \
  catch (const std::exception& e) { return fail(FX_E_INVALID, e.what()); }

#define HIP_OK(expr)                                                                                  \
  do {                                                                                                \
    hipError_t e__ = (expr);                                                                          \
    if (e__ != hipSuccess) return fail(FX_E_HIP, std::string(#expr) + ": " + hipGetErrorString(e__)); \
  } while (0)

int add_value(fx_region* reg, const fx::Value& v, int* id) {
  if (!reg || !id) return fail(FX_E_INVALID, "null argument");
  if (reg->r.finalized) return fail(FX_E_INVALID, "region already finalized");
  *id = reg->r.add(v);
  return FX_OK;
}

}  // namespace

extern "C" {

const char* fx_last_error(void) { return g_err.c_str(); }
int fx_api_version(void) { return FX_API_VERSION; }

int fx_region_create(int parallel_degree, int is_parallel_map, fx_region** out) {
  if (!out) return fail(FX_E_INVALID, "null out");
  if (parallel_degree < 1) return fail(FX_E_INVALID, "parallel_degree must be >= 1");
  fx_region* r = new fx_region();
  r->r.degree = parallel_degree;
  r->r.is_map = is_parallel_map != 0;
  *out = r;
  return FX_OK;
}

void fx_region_destroy(fx_region* r) {
  if (!r) return;
  for (auto& kv : r->r.plans) {
    if (kv.second->dev_blob) (void)hipFree(kv.second->dev_blob);
    for (auto& st : kv.second->status)
      if (st.ptr) (void)hipFree(st.ptr);
  }
  delete r;
}

int fx_region_input_tensor(fx_region* reg, int dtype, int rank, int per_task, int* id) {
  if (!reg) return fail(FX_E_INVALID, "null region");
  if (fx::dtype_size(dtype) == 0) return fail(FX_E_UNSUPPORTED, "unsupported tensor dtype");
  fx::Value v;
  v.kind = fx::VK_TENSOR;
  v.prod = fx::P_INPUT;
  v.dtype = dtype;
  v.rank = rank;
  v.per_task = per_task != 0;
  v.input_index = (int)reg->r.inputs.size();
  int rc = add_value(reg, v, id);
  if (rc == FX_OK) reg->r.inputs.push_back(*id);
  return rc;
}

int fx_region_input_scalar(fx_region* reg, int kind, int per_task, int* id) {
  if (!reg) return fail(FX_E_INVALID, "null region");
  if (kind < 1 || kind > 3) return fail(FX_E_INVALID, "scalar kind must be 1 (int), 2 (float) or 3 (bool)");
  fx::Value v;
  v.kind = kind == 1 ? fx::VK_INT : (kind == 2 ? fx::VK_FLOAT : fx::VK_BOOL);
  v.prod = fx::P_INPUT;
  v.per_task = per_task != 0;
  v.input_index = (int)reg->r.inputs.size();
  int rc = add_value(reg, v, id);
  if (rc == FX_OK) reg->r.inputs.push_back(*id);
  return rc;
}

int fx_region_task_index(fx_region* reg, int* id) {
  fx::Value v;
  v.kind = fx::VK_INT;
  v.prod = fx::P_TASK;
  return add_value(reg, v, id);
}

int fx_region_loop_var(fx_region* reg, int* id) {
  fx::Value v;
  v.kind = fx::VK_INT;
  v.prod = fx::P_LOOPVAR;
  return add_value(reg, v, id);
}

int fx_region_const_int(fx_region* reg, int64_t x, int* id) {
  fx::Value v;
  v.kind = fx::VK_INT;
  v.ival = x;
  return add_value(reg, v, id);
}
int fx_region_const_float(fx_region* reg, double x, int* id) {
  fx::Value v;
  v.kind = fx::VK_FLOAT;
  v.fval = x;
  return add_value(reg, v, id);
}
int fx_region_const_bool(fx_region* reg, int x, int* id) {
  fx::Value v;
  v.kind = fx::VK_BOOL;
  v.ival = x != 0;
  return add_value(reg, v, id);
}
int fx_region_const_none(fx_region* reg, int* id) {
  fx::Value v;
  v.kind = fx::VK_NONE;
  return add_value(reg, v, id);
}

static int add_list(fx_region* reg, const int* ids, int n, fx::VKind kind, fx::VKind elem, int* id) {
  if (!reg || (n > 0 && !ids)) return fail(FX_E_INVALID, "null argument");
  fx::Value v;
  v.kind = kind;
  v.prod = fx::P_LIST;
  for (int i = 0; i < n; ++i) {
    if (ids[i] < 0 || ids[i] >= (int)reg->r.vals.size()) return fail(FX_E_INVALID, "bad value id in list");
    fx::VKind k = reg->r.vals[ids[i]].kind;
    if (elem == fx::VK_INT ? !(k == fx::VK_INT || k == fx::VK_BOOL) : k != elem)
      return fail(FX_E_INVALID, "list element of the wrong kind");
    v.args.push_back(ids[i]);
  }
  return add_value(reg, v, id);
}
int fx_region_int_list(fx_region* reg, const int* ids, int n, int* id) {
  return add_list(reg, ids, n, fx::VK_INT_LIST, fx::VK_INT, id);
}
int fx_region_tensor_list(fx_region* reg, const int* ids, int n, int* id) {
  return add_list(reg, ids, n, fx::VK_TENSOR_LIST, fx::VK_TENSOR, id);
}

int fx_region_op(fx_region* reg, int opcode, const int* arg_ids, int n_args, int out_dtype, int* id) {
  if (!reg || !id || (n_args > 0 && !arg_ids)) return fail(FX_E_INVALID, "null argument");
  if (reg->r.finalized) return fail(FX_E_INVALID, "region already finalized");
  FX_TRY
  std::vector<int> args(arg_ids, arg_ids + n_args);
  *id = reg->r.addOp(opcode, args, out_dtype);
  return FX_OK;
  FX_CATCH
}

int fx_region_output(fx_region* reg, int value_id) {
  if (!reg) return fail(FX_E_INVALID, "null region");
  if (reg->r.finalized) return fail(FX_E_INVALID, "region already finalized");
  if (value_id < 0 || value_id >= (int)reg->r.vals.size() || reg->r.vals[value_id].kind != fx::VK_TENSOR)
    return fail(FX_E_INVALID, "output must be a tensor value");
  reg->r.outputs.push_back(value_id);
  return FX_OK;
}

int fx_region_compact_rows(fx_region* reg, int mask_value_id) {
  if (!reg) return fail(FX_E_INVALID, "null region");
  if (reg->r.finalized) return fail(FX_E_INVALID, "region already finalized");
  if (mask_value_id < 0 || mask_value_id >= (int)reg->r.vals.size() ||
      reg->r.vals[mask_value_id].kind != fx::VK_TENSOR)
    return fail(FX_E_INVALID, "mask must be a tensor value");
  reg->r.mask = mask_value_id;
  return FX_OK;
}

int fx_region_finalize(fx_region* reg) {
  if (!reg) return fail(FX_E_INVALID, "null region");
  if (reg->r.outputs.empty()) return fail(FX_E_INVALID, "region has no outputs");
  reg->r.finalized = true;
  return FX_OK;
}

// ---- specialised kernels ----
static std::atomic<int> g_specialize{[] {
  const char* e = getenv("FXHIP_SPECIALIZE");
  return (e && e[0] == '0') ? 0 : 1;
}()};
// ---- streaming compaction: process-wide switches ----
static std::atomic<int> g_stream_mode{[] {
  const char* e = getenv("FXHIP_STREAM");
  return (e && e[0] == '1') ? 1 : 0;
}()};
// ---- detection-head kernel (fx_head.h): on unless FXHIP_HEAD=0 ----
static std::atomic<int> g_head_mode{[] {
  const char* e = getenv("FXHIP_HEAD");
  return (e && e[0] == '0') ? 0 : 1;
}()};
// ---- generated row-stream kernels (fx_rs.h): on unless FXHIP_ROWSTREAM=0 ----
static std::atomic<int> g_rs_mode{[] {
  const char* e = getenv("FXHIP_ROWSTREAM");
  return (e && e[0] == '0') ? 0 : 1;
}()};
static std::atomic<uint32_t> g_stream_spin{[] {
  const char* e = getenv("FXHIP_STREAM_SPIN");
  return e ? (uint32_t)strtoul(e, nullptr, 10) : 4000u;
}()};
static std::atomic<uint32_t> g_totals_spin_us{2000u};   // microseconds that fx_region_wait_totals polls from the host before it blocks in the stream
static std::atomic<uint32_t> g_lstm_spin{1000000u};   // polls of a wait of fx_lstm_stack before it is given up
static std::mutex g_dump_mu;
static std::string g_dump_dir;
static int g_dump_what = 3;   // bit 0: program tables (fx_spec_*), bit 1: row-stream units (fx_rs_*)

static std::atomic<uint64_t> g_launches{0}, g_spec_launches{0};

static const FxSpecKernels* spec_of(const fx::Plan* p) {
  if (!g_specialize.load(std::memory_order_relaxed) || p->spec_key == 0) return nullptr;
  return fx_spec_find(p->spec_key);
}

// With a dump directory set, every plan that has no specialised kernels linked in leaves
// the translation unit that would specialise it there (one file per key).
static void dump_spec_source(const fx::Plan* p) {
  std::string dir;
  int what = 3;
  {
    std::lock_guard<std::mutex> g(g_dump_mu);
    dir = g_dump_dir;
    what = g_dump_what;
  }
  if (!dir.empty() && (what & 2) && p->rs.ok && !fx_rs_find(p->rs.key)) {
    char rname[64];
    snprintf(rname, sizeof(rname), "/fx_rs_%016llx.hip", (unsigned long long)p->rs.key);
    const std::string rpath = dir + rname;
    if (FILE* f = fopen(rpath.c_str(), "r")) {
      fclose(f);
    } else {
      std::string label = "row compaction, outputs of task 0:";
      for (size_t o = 0; o < p->out_shape.size(); ++o) {
        label += " [";
        const auto& sh = p->out_shape[o][0];
        for (size_t d = 0; d < sh.size(); ++d) label += (d ? "," : "") + std::to_string(sh[d]);
        label += "]";
      }
      const std::string src = fx::rs_source(*p, label);
      if (FILE* f = fopen(rpath.c_str(), "w")) {
        fwrite(src.data(), 1, src.size(), f);
        fclose(f);
      }
    }
  }
  if (dir.empty() || !(what & 1) || p->spec_key == 0 || fx_spec_find(p->spec_key)) return;
  char name[64];
  snprintf(name, sizeof(name), "/fx_spec_%016llx.hip", (unsigned long long)p->spec_key);
  const std::string path = dir + name;
  if (FILE* f = fopen(path.c_str(), "r")) { fclose(f); return; }
  // label: what the plan computes, in shapes
  std::string label = p->mode == FX_MODE_COMPACT ? "row compaction, " : "dense, ";
  label += std::to_string(p->region->degree) + " task(s), outputs of task 0:";
  for (size_t o = 0; o < p->out_shape.size(); ++o) {
    label += " [";
    const auto& sh = p->out_shape[o][0];
    for (size_t d = 0; d < sh.size(); ++d) label += (d ? "," : "") + std::to_string(sh[d]);
    label += "]";
  }
  const std::string src = fx::spec_source(*p, label);
  if (FILE* f = fopen(path.c_str(), "w")) {
    fwrite(src.data(), 1, src.size(), f);
    fclose(f);
  }
}

int fx_region_plan(fx_region* reg, const fx_arg* args, int n_args, const fx_plan** plan) {
  if (!reg || !plan || (n_args > 0 && !args)) return fail(FX_E_INVALID, "null argument");
  FX_TRY
  std::lock_guard<std::mutex> g(reg->mu);
  const fx::Plan* p = fx::plan_region(reg->r, args, n_args);
  *plan = reinterpret_cast<const fx_plan*>(p);
  dump_spec_source(p);
  return FX_OK;
  FX_CATCH
}

static const fx::Plan* P(const fx_plan* p) { return reinterpret_cast<const fx::Plan*>(p); }

void fx_set_specialization(int on) { g_specialize.store(on ? 1 : 0, std::memory_order_relaxed); }
int fx_specialization_count(void) { return fx_spec_count(); }
int fx_plan_specialized(const fx_plan* p) { return (p && spec_of(P(p))) ? 1 : 0; }
uint64_t fx_plan_spec_key(const fx_plan* p) { return p ? P(p)->spec_key : 0; }

int fx_plan_spec_source(const fx_plan* p, const char* label, char* buf, size_t cap) {
  if (!p || !buf || cap == 0) return fail(FX_E_INVALID, "null argument");
  FX_TRY
  std::string s = fx::spec_source(*P(p), label ? label : "");
  size_t n = std::min(cap - 1, s.size());
  memcpy(buf, s.data(), n);
  buf[n] = 0;
  return (int)s.size();
  FX_CATCH
}

void fx_launch_stats(uint64_t* total, uint64_t* specialised) {
  if (total) *total = g_launches.load(std::memory_order_relaxed);
  if (specialised) *specialised = g_spec_launches.load(std::memory_order_relaxed);
}

int fx_spec_dump_dir(const char* dir) {
  std::lock_guard<std::mutex> g(g_dump_mu);
  g_dump_dir = dir ? dir : "";
  return FX_OK;
}
int fx_spec_dump_what(int what) {
  std::lock_guard<std::mutex> g(g_dump_mu);
  const int before = g_dump_what;
  g_dump_what = what & 3;
  return before;
}

int fx_plan_num_outputs(const fx_plan* p) { return p ? (int)P(p)->out_dtype.size() : 0; }

int fx_plan_output(const fx_plan* p, int out_idx, int task, int32_t* dtype, int32_t* rank, int64_t* sizes) {
  if (!p) return fail(FX_E_INVALID, "null plan");
  const fx::Plan* pl = P(p);
  if (out_idx < 0 || out_idx >= (int)pl->out_dtype.size() || task < 0 || task >= pl->region->degree)
    return fail(FX_E_INVALID, "output/task index out of range");
  const auto& s = pl->out_shape[out_idx][task];
  if (dtype) *dtype = pl->out_dtype[out_idx];
  if (rank) *rank = (int32_t)s.size();
  if (sizes)
    for (size_t i = 0; i < s.size(); ++i) sizes[i] = s[i];
  return FX_OK;
}

size_t fx_plan_scratch_bytes(const fx_plan* p) { return p ? P(p)->scratch_bytes : 0; }
static bool stream_active(const fx::Plan* pl, const FxSpecKernels* spec);
static const FxSpecKernels* spec_of(const fx::Plan* p);
static const FxRsKernel* rs_of(const fx::Plan* pl);
static void rs_fill_params(const fx::Plan* pl, FxRsLaunch* rl, const FxRsKernel* kern);
static bool head_active(const fx::Plan* pl) {
  // (with compiled kernels switched off, fx_set_specialization(0), everything runs in the interpreter)
  return pl->mode == FX_MODE_COMPACT && pl->head.ok && g_head_mode.load(std::memory_order_relaxed) != 0 &&
         g_specialize.load(std::memory_order_relaxed) != 0;
}
static bool cmap_active(const fx::Plan* pl) {
  return pl->mode == FX_MODE_COMPACT && pl->cmap.ok && g_head_mode.load(std::memory_order_relaxed) != 0 &&
         g_specialize.load(std::memory_order_relaxed) != 0;
}
void fx_set_head_kernel(int on) { g_head_mode.store(on ? 1 : 0, std::memory_order_relaxed); }
int fx_plan_head_info(const fx_plan* p, int64_t* out, int cap) {
  if (!p || !out || cap < 8) return fail(FX_E_INVALID, "fx_plan_head_info: out[>=8] required");
  const FxHeadInfo& hi = P(p)->head;
  const FxCmapInfo& ci = P(p)->cmap;
  if (ci.ok || (!hi.ok && ci.norm_hash && !hi.norm_hash)) {
    out[0] = ci.ok ? 2 : 0;
    out[1] = cmap_active(P(p)) ? 1 : 0;
    out[2] = (int64_t)(ci.norm_hash & 0xffffffffull);
    out[3] = (int64_t)(ci.norm_hash >> 32);
    out[4] = ci.n_tasks;
    out[5] = ci.C;
    out[6] = ci.n_rows;
    out[7] = ci.first;
    return FX_OK;
  }
  out[0] = hi.ok ? 1 : 0;
  out[1] = (head_active(P(p)) && !rs_of(P(p))) ? 1 : 0;
  out[2] = (int64_t)(hi.norm_hash & 0xffffffffull);
  out[3] = (int64_t)(hi.norm_hash >> 32);
  out[4] = hi.C;
  out[5] = hi.S;
  out[6] = hi.n_rows;
  out[7] = hi.n_tasks;
  return FX_OK;
}
void fx_set_rowstream(int on) { g_rs_mode.store(on == 2 ? 2 : (on ? 1 : 0), std::memory_order_relaxed); }
int fx_rowstream_count(void) { return fx_rs_count(); }
int fx_plan_rowstream_info(const fx_plan* p, int64_t* out, int cap) {
  if (!p || !out || cap < 8) return fail(FX_E_INVALID, "fx_plan_rowstream_info: out[>=8] required");
  const FxRsInfo& ri = P(p)->rs;
  out[0] = ri.ok ? 1 : 0;
  out[1] = rs_of(P(p)) ? 1 : 0;
  out[2] = (int64_t)(ri.key & 0xffffffffull);
  out[3] = (int64_t)(ri.key >> 32);
  out[4] = ri.S;
  out[5] = ri.n_rows;
  out[6] = ri.n_tasks;
  out[7] = ri.n_in;
  return FX_OK;
}
int fx_plan_rowstream_why(const fx_plan* p, char* buf, size_t cap) {
  if (!p || !buf || cap == 0) return fail(FX_E_INVALID, "null argument");
  const std::string& s = P(p)->rs.why;
  const size_t n = std::min(cap - 1, s.size());
  memcpy(buf, s.data(), n);
  buf[n] = 0;
  return (int)s.size();
}
int fx_plan_rowstream_launch(const fx_plan* p, uint32_t chunk_rows, uint32_t sub_rows, void* out, size_t cap) {
  if (!p || !out || cap < sizeof(FxRsLaunch)) return fail(FX_E_INVALID, "fx_plan_rowstream_launch: out too small");
  if (!P(p)->rs.ok) return fail(FX_E_UNSUPPORTED, "this plan has no row-stream form: " + P(p)->rs.why);
  FxRsLaunch rl;
  rs_fill_params(P(p), &rl, nullptr);
  if (chunk_rows == 0 || chunk_rows > FX_BLOCK || sub_rows == 0 || sub_rows > rl.sub_rows)
    return fail(FX_E_INVALID, "fx_plan_rowstream_launch: chunk rows 1.." + std::to_string(FX_BLOCK) + ", sub-tile rows 1.." + std::to_string(rl.sub_rows));
  rl.chunk_rows = chunk_rows;
  rl.chunks = (rl.n_rows + chunk_rows - 1) / chunk_rows;
  rl.sub_rows = sub_rows;
  fx_rs_finish_geometry(&rl);
  memcpy(out, &rl, sizeof(rl));
  return (int)sizeof(rl);
}
int fx_plan_rowstream_source(const fx_plan* p, const char* label, char* buf, size_t cap) {
  if (!p || !buf || cap == 0) return fail(FX_E_INVALID, "null argument");
  FX_TRY
  std::string s = fx::rs_source(*P(p), label ? label : "");
  size_t n = std::min(cap - 1, s.size());
  memcpy(buf, s.data(), n);
  buf[n] = 0;
  return (int)s.size();
  FX_CATCH
}
int fx_plan_launches(const fx_plan* p) {
  if (!p) return 0;
  if (rs_of(P(p)) || head_active(P(p)) || cmap_active(P(p))) return 1;
  if (P(p)->mode == FX_MODE_COMPACT && stream_active(P(p), spec_of(P(p)))) return P(p)->stream.grid > 0 ? 1 : 0;
  return P(p)->launches;
}
int fx_plan_streaming(const fx_plan* p) {
  return (p && P(p)->mode == FX_MODE_COMPACT && !rs_of(P(p)) && !head_active(P(p)) && !cmap_active(P(p)) && stream_active(P(p), spec_of(P(p)))) ? 1 : 0;
}
int fx_plan_stream_info(const fx_plan* p, int64_t* out, int cap) {
  if (!p || !out || cap < 8) return fail(FX_E_INVALID, "fx_plan_stream_info: out[>=8] required");
  const fx::StreamInfo& si = P(p)->stream;
  out[0] = si.ok ? 1 : 0;
  out[1] = si.tile_rows;
  out[2] = si.tiles_per_task;
  out[3] = si.grid;
  out[4] = si.win_stride;
  out[5] = si.win_tcoef;
  out[6] = si.win_lo;
  out[7] = si.win_span;
  return FX_OK;
}
void fx_set_streaming(int on) { g_stream_mode.store(on ? 1 : 0, std::memory_order_relaxed); }
void fx_set_stream_spin_limit(uint32_t polls) { g_stream_spin.store(polls, std::memory_order_relaxed); }
int64_t fx_plan_algorithmic_bytes(const fx_plan* p) { return p ? P(p)->alg_bytes : 0; }

int fx_plan_blob(const fx_plan* p, const uint32_t** words, size_t* n_words) {
  if (!p || !words || !n_words) return fail(FX_E_INVALID, "null argument");
  *words = P(p)->blob.data();
  *n_words = P(p)->blob.size();
  return FX_OK;
}

int fx_plan_disasm(const fx_plan* p, char* buf, size_t cap) {
  if (!p || !buf || cap == 0) return fail(FX_E_INVALID, "null argument");
  std::string s = fx::disasm(*P(p));
  size_t n = std::min(cap - 1, s.size());
  memcpy(buf, s.data(), n);
  buf[n] = 0;
  return (int)s.size();
}

int fx_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) return 0;
  return n;
}

// Error word of checked int64 loads (fx_bytecode.h FX_I64): one word of pinned host memory
// that every device can write; without a device (host-only marshalling for the emulator) a
// plain word stands in.
static std::mutex g_err_mu;
static uint32_t* g_err_pinned = nullptr;
static uint32_t g_err_plain = 0;
static uint32_t* err_word(bool pinned) {
  std::lock_guard<std::mutex> g(g_err_mu);
  if (g_err_pinned) return g_err_pinned;
  if (!pinned) return &g_err_plain;
  void* p = nullptr;
  if (hipHostMalloc(&p, 64, hipHostMallocPortable | hipHostMallocMapped) != hipSuccess) return nullptr;
  g_err_pinned = (uint32_t*)p;
  *g_err_pinned = 0;
  return g_err_pinned;
}

int fx_async_error(int clear) {
  std::lock_guard<std::mutex> g(g_err_mu);
  uint32_t v = g_err_plain;
  if (g_err_pinned) v |= *(volatile uint32_t*)g_err_pinned;
  if (clear) {
    g_err_plain = 0;
    if (g_err_pinned) *(volatile uint32_t*)g_err_pinned = 0;
  }
  return (int)v;
}

void fx_async_error_report(int bits) {
  std::lock_guard<std::mutex> g(g_err_mu);
  g_err_plain |= (uint32_t)bits;
}
int fx_async_error_take(int mask) {
  std::lock_guard<std::mutex> g(g_err_mu);
  uint32_t v = g_err_plain;
  if (g_err_pinned) v |= *(volatile uint32_t*)g_err_pinned;
  g_err_plain &= ~(uint32_t)mask;
  if (g_err_pinned) *(volatile uint32_t*)g_err_pinned = *(volatile uint32_t*)g_err_pinned & ~(uint32_t)mask;
  return (int)(v & (uint32_t)mask);
}

// Fill the by-value dynamic block.  Exposed (without launching) so that host
// tests can check the marshalling.
// `safe`: a device address that can always be read.  Kernels clamp the address of
// an element that is not live to element 0 of its buffer, so a tensor without
// elements (whose pointer may be null) is given this address instead.
static int fill_tables(const fx::Plan* pl, const fx_arg* args, void* const* out_ptrs, void* scratch,
                       uint32_t* totals_host, const void* safe, uint64_t* p_out, uint32_t* s_out, const void* status);
static int fill_dyn(const fx::Plan* pl, const fx_arg* args, void* const* out_ptrs, void* scratch,
                    uint32_t* totals_host, const void* safe, FxDyn* dyn, const void* status = nullptr) {
  if (pl->wide) return fail(FX_E_LIMIT, "the tables of this plan do not fit the kernel argument block (a map of many tasks): fx_region_run uploads them");
  return fill_tables(pl, args, out_ptrs, scratch, totals_host, safe, dyn->p, dyn->s, status);
}
static int fill_tables(const fx::Plan* pl, const fx_arg* args, void* const* out_ptrs, void* scratch,
                       uint32_t* totals_host, const void* safe, uint64_t* p_out, uint32_t* s_out, const void* status) {
  const fx::Region& R = *pl->region;
  const int T = R.degree;
  auto ptr_of = [&](const fx::PtrSrc& s, int task) -> uint64_t {
    switch (s.kind) {
      case fx::PtrSrc::INPUT: {
        bool per_task = R.vals[R.inputs[s.index]].per_task;
        const fx_arg& a = args[pl->arg_base[s.index] + (per_task ? task : 0)];
        bool empty = a.ptr == nullptr;
        for (int d = 0; d < a.rank; ++d) empty = empty || a.sizes[d] == 0;
        return (uint64_t)(uintptr_t)((empty && safe) ? safe : a.ptr);
      }
      case fx::PtrSrc::OUTPUT: return (uint64_t)(uintptr_t)out_ptrs[s.index * T + task];
      case fx::PtrSrc::FLAGS: return (uint64_t)(uintptr_t)((char*)scratch + pl->flags_off);
      case fx::PtrSrc::COUNTS: return (uint64_t)(uintptr_t)((char*)scratch + pl->counts_off);
      case fx::PtrSrc::TOTALS: return (uint64_t)(uintptr_t)totals_host;
      case fx::PtrSrc::ERRWORD: return (uint64_t)(uintptr_t)err_word(safe != nullptr);
      case fx::PtrSrc::STATUS: return (uint64_t)(uintptr_t)status;
    }
    return 0;
  };
  bool scalar_overflow = false;
  auto scal_of = [&](const fx::ScalSrc& s, int task) -> uint32_t {
    const fx::Value& v = R.vals[R.inputs[s.input]];
    const fx_arg& a = args[pl->arg_base[s.input] + (v.per_task ? task : 0)];
    double x = v.kind == fx::VK_FLOAT ? a.fval : (double)a.ival;
    uint32_t u;
    if (s.as_float) {
      float f = (float)x;  // double -> float like graph_builder.cpp:850-854
      memcpy(&u, &f, 4);
    } else {
      const int64_t i = v.kind == fx::VK_FLOAT ? (int64_t)a.fval : a.ival;
      scalar_overflow = scalar_overflow || i != (int64_t)(int32_t)i;
      u = (uint32_t)(int32_t)i;
    }
    return u;
  };
  size_t np = pl->sptr.size(), ntp = pl->tptr.size(), ns = pl->sscal.size(), nts = pl->tscal.size();
  for (size_t i = 0; i < np; ++i) p_out[i] = ptr_of(pl->sptr[i], 0);
  for (int t = 0; t < T; ++t)
    for (size_t i = 0; i < ntp; ++i) p_out[np + t * ntp + i] = ptr_of(pl->tptr[i], t);
  for (size_t i = 0; i < ns; ++i) s_out[i] = scal_of(pl->sscal[i], 0);
  for (int t = 0; t < T; ++t)
    for (size_t i = 0; i < nts; ++i) s_out[ns + t * nts + i] = scal_of(pl->tscal[i], t);
  if (scalar_overflow) return fail(FX_E_LIMIT, "an integer scalar argument is outside 32 bits (integer arithmetic in regions is 32-bit)");
  if (pl->uses_guard && safe && !err_word(true)) return fail(FX_E_HIP, "no pinned memory for the error word");
  return FX_OK;
}

int fx_region_marshal(fx_region* reg, const fx_plan* plan, const fx_arg* args, int n_args, void* const* out_ptrs,
                      void* scratch, uint32_t* totals_host, void* dyn_out, size_t dyn_cap) {
  if (!reg || !plan || !out_ptrs || !dyn_out) return fail(FX_E_INVALID, "null argument");
  const fx::Plan* pl = P(plan);
  if (pl->region != &reg->r) return fail(FX_E_INVALID, "plan does not belong to this region");
  if (n_args != pl->n_args) return fail(FX_E_INVALID, "argument count differs from the plan");
  if (dyn_cap < sizeof(FxDyn)) return fail(FX_E_INVALID, "dyn_out too small");
  memset(dyn_out, 0, sizeof(FxDyn));
  return fill_dyn(pl, args, out_ptrs, scratch, totals_host, nullptr, (FxDyn*)dyn_out);
}

size_t fx_dyn_bytes(void) { return sizeof(FxDyn); }

int fx_plan_table_sizes(const fx_plan* plan, size_t* n_pointers, size_t* n_scalars, int* uploaded) {
  if (!plan) return fail(FX_E_INVALID, "null argument");
  const fx::Plan* pl = P(plan);
  const size_t T = (size_t)pl->region->degree;
  if (n_pointers) *n_pointers = pl->sptr.size() + pl->tptr.size() * T;
  if (n_scalars) *n_scalars = pl->sscal.size() + pl->tscal.size() * T;
  if (uploaded) *uploaded = pl->wide ? 1 : 0;
  return FX_OK;
}

int fx_region_marshal_tables(fx_region* reg, const fx_plan* plan, const fx_arg* args, int n_args, void* const* out_ptrs,
                             void* scratch, uint32_t* totals_host, uint64_t* pointers, size_t pointer_cap,
                             uint32_t* scalars, size_t scalar_cap) {
  if (!reg || !plan || !out_ptrs || !pointers || !scalars) return fail(FX_E_INVALID, "null argument");
  const fx::Plan* pl = P(plan);
  if (pl->region != &reg->r) return fail(FX_E_INVALID, "plan does not belong to this region");
  if (n_args != pl->n_args) return fail(FX_E_INVALID, "argument count differs from the plan");
  size_t np = 0, ns = 0;
  fx_plan_table_sizes(plan, &np, &ns, nullptr);
  if (pointer_cap < np || scalar_cap < ns) return fail(FX_E_INVALID, "tables too small (fx_plan_table_sizes)");
  return fill_tables(pl, args, out_ptrs, scratch, totals_host, nullptr, pointers, scalars, nullptr);
}

// ---- streaming compaction: per-stream status words ----
#define FX_STREAM_LDS_LIMIT 64000u   // 64 KiB less the kernel's static tables
#define FX_EPOCH_MAX ((1u << 23) - 1u)

// Lean dense kernel (fx_spec.h): on unless switched off (tests compare it with the general kernel).
static std::atomic<int> g_dense_lean{[] {
  const char* e = getenv("FXHIP_DENSE_LEAN");
  return (e && e[0] == '0') ? 0 : 1;
}()};
static const FxLeanArgs* lean_of(const fx::Plan* pl) {
  return g_dense_lean.load(std::memory_order_relaxed) ? &pl->lean : nullptr;
}

int fx_plan_dense_lean(const fx_plan* p) {
  if (!p) return 0;
  const fx::Plan* pl = P(p);
  return (pl->mode == FX_MODE_DENSE && lean_of(pl) && pl->lean.n_outs != 0 && fx_spec_has_lean(spec_of(pl))) ? 1 : 0;
}
void fx_set_dense_lean(int on) { g_dense_lean.store(on ? 1 : 0, std::memory_order_relaxed); }

static FxLaunchInfo launch_info(const fx::Plan* pl) {
  const fx::Region& R = *pl->region;
  FxLaunchInfo li;
  memset(&li, 0, sizeof(li));
  li.blob_words = (uint32_t)pl->blob.size();
  li.n_p = (uint32_t)(pl->sptr.size() + pl->tptr.size() * (size_t)R.degree);
  li.n_s = (uint32_t)(pl->sscal.size() + pl->tscal.size() * (size_t)R.degree);
  li.n_temps = pl->n_temps;
  li.total_units = pl->mode == FX_MODE_DENSE ? pl->grid : 0;
  if (pl->stream.ok) {
    const fx::StreamInfo& si = pl->stream;
    li.win_words = si.win_words;
    li.s_tiles = si.tiles_per_task;
    li.s_rows = si.rows;
    li.s_tile_rows = si.tile_rows;
    li.s_win_slot = si.win_slot;
    li.s_win_stride = si.win_stride;
    li.s_win_tcoef = si.win_tcoef;
    li.s_win_lo = si.win_lo;
    li.s_win_span = si.win_span;
    li.n_sptr = (uint32_t)pl->sptr.size();
    li.n_tptr = (uint32_t)pl->tptr.size();
    li.spin_limit = g_stream_spin.load(std::memory_order_relaxed);
    li.n_side = si.n_side;
    for (int i = 0; i < 2; ++i) {
      li.side_slot[i] = si.side_slot[i];
      li.side_stride[i] = si.side_stride[i];
      li.side_tcoef[i] = si.side_tcoef[i];
      li.side_lo[i] = si.side_lo[i];
      li.side_span[i] = si.side_span[i];
      li.side_words[i] = si.side_words[i];
    }
  }
  return li;
}

// does a call of this plan run as one streaming kernel (with the kernels it would use now)?
static bool stream_active(const fx::Plan* pl, const FxSpecKernels* spec) {
  if (!pl->stream.ok || !g_stream_mode.load(std::memory_order_relaxed)) return false;
  const bool compiled = spec && fx_spec_has_stream(spec);
  return fx_stream_lds_bytes(launch_info(pl), compiled) <= FX_STREAM_LDS_LIMIT;
}

// persistent workgroups: as many as stay resident together (two per CU: the kernel keeps the
// next tile's rows in registers), striding over the tiles
#define FX_STREAM_WG_PER_CU 2u
static uint32_t stream_grid(const fx::Plan* pl) { return std::min<uint32_t>(pl->stream.grid, 256u * FX_STREAM_WG_PER_CU); }

// Status words of `pl` for launches on `stream` (created on first use, at most four streams per
// plan: calls on further streams take the two-pass form) and the epoch of the next call.
static int status_words(fx_region* reg, std::vector<fx::Plan::Status>& list, size_t words, hipStream_t stream, int dev,
                        void** ptr, uint32_t* epoch, int n_epochs, uint32_t epoch_max = FX_EPOCH_MAX) {
  std::lock_guard<std::mutex> g(reg->mu);
  fx::Plan::Status* st = nullptr;
  for (auto& s : list)
    if (s.stream == (void*)stream && s.dev == dev) st = &s;
  const size_t bytes = std::max<size_t>(words, 1) * 4;
  if (!st) {
    if (list.size() >= 4) { *ptr = nullptr; return FX_OK; }
    void* d = nullptr;
    HIP_OK(hipMalloc(&d, bytes));
    HIP_OK(hipMemset(d, 0, bytes));
    list.push_back({(void*)stream, d, 0u, dev});
    st = &list.back();
  }
  if (st->epoch + (uint32_t)n_epochs >= epoch_max) {
    // the tags wrap: clear the words behind everything already queued on the stream
    HIP_OK(hipMemsetAsync(st->ptr, 0, bytes, stream));
    st->epoch = 0;
  }
  *ptr = st->ptr;
  *epoch = st->epoch + 1;
  st->epoch += (uint32_t)n_epochs;
  return FX_OK;
}
static int stream_status(fx_region* reg, fx::Plan* pl, hipStream_t stream, int dev, void** ptr, uint32_t* epoch,
                         int n_epochs) {
  return status_words(reg, pl->status, pl->stream.grid, stream, dev, ptr, epoch, n_epochs);
}

// ---- detection-head kernel: geometry of a launch ----
// Rows of a sub-tile: what FX_HEAD_KV 128-bit loads per lane carry, at most FX_HEAD_SUB.
static uint32_t head_sub_rows(const FxHeadInfo& hi) {
  const uint32_t cap = (FX_HEAD_KV * FX_BLOCK * 4u - 6u) / hi.S;
  return std::min<uint32_t>(FX_HEAD_SUB, cap);
}
static size_t head_status_words(const FxHeadInfo& hi) {
  const uint32_t min_chunk = std::min<uint32_t>(FX_HEAD_MIN_CHUNK, std::max<uint32_t>(hi.n_rows, 1u));
  return (size_t)hi.n_tasks * ((hi.n_rows + min_chunk - 1) / min_chunk);
}
static bool head_fits(const fx::Plan* pl) {
  // a sub-tile of at least 8 rows, and counts of up to FX_BLOCK rows in a status word
  return head_active(pl) && head_sub_rows(pl->head) >= 8u;
}
// Every image's rows are dealt to its workgroups in equal runs, as few workgroups as give every
// resident slot of the device one (more only when a chunk would exceed FX_BLOCK rows, fewer when
// it would fall below FX_HEAD_MIN_CHUNK).
static int head_launch_info(fx::Plan* pl, FxHeadLaunch* hl) {
  const FxHeadInfo& hi = pl->head;
  memset(hl, 0, sizeof(*hl));
  hl->n_rows = hi.n_rows;
  hl->n_tasks = hi.n_tasks;
  hl->sub_rows = head_sub_rows(hi);
  hl->S = hi.S;
  hl->C = hi.C;
  fx_fastdiv_make(hi.C / 4u, &hl->g_magic, &hl->g_shift);
  hl->thr_bits = hi.thr_bits;
  hl->spin_limit = g_stream_spin.load(std::memory_order_relaxed);
  hl->n_sptr = (uint32_t)pl->sptr.size();
  hl->n_tptr = (uint32_t)pl->tptr.size();
  hl->pred_slot = hi.pred_slot;
  hl->anc_slot = hi.anc_slot;
  hl->strd_slot = hi.strd_slot;
  hl->pred_tcoef = hi.pred_tcoef;
  hl->anc_tcoef = hi.anc_tcoef;
  hl->strd_tcoef = hi.strd_tcoef;
  hl->folded = hi.folded ? 1u : 0u;
  hl->half_slot = hi.half_slot;
  hl->half_tcoef = hi.half_tcoef;
  for (int k = 0; k < 3; ++k) {
    hl->out_slot[k] = hi.out_slot[k];
    hl->out_tstride[k] = hi.out_tstride[k];
  }
  if (pl->head_resident == 0) {
    // One slot per CU is left free: a launch that needs every slot the occupancy rule allows does
    // not get all of its workgroups placed at once, and the stragglers cost a second round.
    uint32_t wg = 0, per_cu = 1;
    HIP_OK(fx_head_resident(fx_head_lds_bytes(*hl), &wg, &per_cu));
    if (per_cu >= 3) wg -= wg / per_cu;
    pl->head_resident = std::max<uint32_t>(wg, 1u);
  }
  const uint32_t per_task = std::max<uint32_t>(1u, pl->head_resident / std::max<uint32_t>(hi.n_tasks, 1u));
  uint32_t cr = (hi.n_rows + per_task - 1) / per_task;
  const uint32_t min_chunk = std::min<uint32_t>(FX_HEAD_MIN_CHUNK, std::max<uint32_t>(hi.n_rows, 1u));
  cr = std::min<uint32_t>(FX_BLOCK, std::max<uint32_t>(cr, min_chunk));
  hl->chunk_rows = cr;
  hl->chunks = (hi.n_rows + cr - 1) / cr;
  // A launch whose first sub-tiles alone are megabytes of requests floods the memory system: there
  // the counts get a head start (fx_head.hip; neutral on some boxes, 5 us of 26 on others).  A
  // small launch would only lose the time.
  const uint64_t first_bytes = (uint64_t)hl->chunks * hi.n_tasks * std::min<uint32_t>(cr, hl->sub_rows) * hi.S * 4u;
  hl->bulk_delay = first_bytes >= FX_HEAD_FLOOD_BYTES ? FX_HEAD_BULK_DELAY : 0u;
  return FX_OK;
}

// ---- generated row-stream kernels (fx_rs.h): when, and the geometry of a launch ----
// compute units of the current device (256 where there is none: plans are also made without a GPU)
static uint32_t rs_compute_units() {
  static std::atomic<uint32_t> cached{0};
  uint32_t n = cached.load(std::memory_order_relaxed);
  if (n) return n;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) {
    (void)hipGetLastError();
    return 256u;
  }
  cached.store((uint32_t)cus, std::memory_order_relaxed);
  return (uint32_t)cus;
}
static const FxRsKernel* rs_of(const fx::Plan* pl) {
  if (pl->mode != FX_MODE_COMPACT || !pl->rs.ok || !g_rs_mode.load(std::memory_order_relaxed) ||
      !g_specialize.load(std::memory_order_relaxed))
    return nullptr;
  // The workgroups of a launch are persistent: a launch with more chunks than the device holds
  // workgroups gives every workgroup several chunks in turn.  That pays where the tasks stream
  // rows of their own (a batch of images: 64 images 90 us against 161 us on the two passes).  A
  // map of many tasks over the SAME rows (80 classes over 8 732 rows) would stream them once per
  // task, chunk after chunk, and keeps the generic two passes (27.6 us that way against 22.5 us).
  // (fx_set_rowstream(2) takes the kernel all the same)
  const uint64_t chunks = ((uint64_t)pl->rs.n_rows + FX_BLOCK - 1) / FX_BLOCK;
  const bool rows_of_their_own = pl->rs.n_tasks <= 1 || pl->rs.in_tcoef[0] != 0 || (pl->rs.in_slot[0] & FX_SLOT_TASK) != 0;
  if (g_rs_mode.load(std::memory_order_relaxed) != 2 && !rows_of_their_own &&
      chunks * pl->rs.n_tasks > (uint64_t)rs_compute_units() * FX_RS_OCC)
    return nullptr;
  const FxRsKernel* k = fx_rs_find(pl->rs.key);
  if (k && pl->wide && !k->fn_wide) return nullptr;
  return (k && k->S == pl->rs.S) ? k : nullptr;
}
// Geometry of a launch.  Rows of a sub-tile: at most FX_RS_SUB and what FX_RS_KV 128-bit loads per
// lane carry.  A workgroup pays about one trip to memory per sub-tile (the next one is asked for
// when the current one has arrived), so the number of sub-tiles per chunk counts first, then how
// full they are: measured on 16 x 10647 rows of 85 elements, chunks of 111 rows in two sub-tiles
// take 23.4 us, in three 25.8 us; with a staged output 167 rows in three sub-tiles of 56 take
// 24.3 us, 134 rows in three of 45 25.2 us, 223 rows in four 26.3 us.  Every candidate sub-tile
// size fixes the LDS of a workgroup, with it the workgroups that are resident together, and with
// them the chunk (every task's rows dealt to as many workgroups as are resident, at least
// FX_RS_MIN_CHUNK rows, at most FX_BLOCK): the candidate with the fewest sub-tiles per chunk
// wins, the larger sub-tile among equals.
static uint32_t rs_env(const char* name) {   // tuning aids: 0 when not set
  const char* e = getenv(name);
  return e ? (uint32_t)strtoul(e, nullptr, 10) : 0u;
}
static uint32_t rs_max_sub_rows(const FxRsInfo& ri, uint32_t kv = FX_RS_KV) {
  return std::min<uint32_t>(FX_RS_SUB, (kv * FX_BLOCK * 4u - 6u) / ri.S);
}
// the window, then the staged outputs (fx_rowstream.h lays them out the same way)
// window, staged outputs, and the chunk's table of side values
static uint32_t rs_lds_bytes(const FxRsInfo& ri, const FxRsKernel* k, uint32_t sub, uint32_t chunk_rows, bool side) {
  return (((sub * ri.S + 3u + 3u) >> 2) + 1u) * 16u + (sub * k->stage_row_words + 8u * k->n_staged) * 4u +
         (side ? chunk_rows * k->side_row_words * 4u : 0u);
}
static size_t rs_status_words(const FxRsInfo& ri) {
  const uint32_t min_chunk = std::min<uint32_t>(FX_RS_MIN_CHUNK, std::max<uint32_t>(ri.n_rows, 1u));
  return (size_t)ri.n_tasks * ((ri.n_rows + min_chunk - 1) / min_chunk);
}
// Every task's rows are dealt to its workgroups in equal runs, as few workgroups as give every
// resident slot of the device one (more only when a chunk would exceed FX_BLOCK rows, fewer when
// it would fall below FX_RS_MIN_CHUNK).
static void rs_fill_params(const fx::Plan* pl, FxRsLaunch* rl, const FxRsKernel* kern = nullptr) {
  const FxRsInfo& ri = pl->rs;
  memset(rl, 0, sizeof(*rl));
  rl->n_rows = ri.n_rows;
  rl->n_tasks = ri.n_tasks;
  rl->sub_rows = rs_max_sub_rows(ri);
  (void)kern;
  rl->spin_limit = g_stream_spin.load(std::memory_order_relaxed);
  rl->n_sptr = (uint32_t)pl->sptr.size();
  rl->n_tptr = (uint32_t)pl->tptr.size();
  rl->n_sscal = (uint32_t)pl->sscal.size();
  rl->n_tscal = (uint32_t)pl->tscal.size();
  for (uint32_t k = 0; k < FX_RS_MAX_IN; ++k) {
    rl->in_slot[k] = ri.in_slot[k];
    rl->in_tcoef[k] = ri.in_tcoef[k];
  }
  for (uint32_t k = 0; k < FX_RS_MAX_OUT; ++k) {
    rl->out_slot[k] = ri.out_slot[k];
    rl->out_tstride[k] = ri.out_tstride[k];
  }
  for (uint32_t k = 0; k < FX_RS_MAX_FIMM; ++k) rl->fimm[k] = ri.fimm[k];
  rl->slot_err = ri.slot_err;
}
static int rs_launch_info(fx::Plan* pl, const FxRsKernel* kern, FxRsLaunch* rl) {
  const FxRsInfo& ri = pl->rs;
  rs_fill_params(pl, rl, kern);
  if (pl->rs_sub_rows == 0) {
    int dev = 0, cus = 0;
    HIP_OK(hipGetDevice(&dev));
    HIP_OK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const uint32_t min_chunk = std::min<uint32_t>(FX_RS_MIN_CHUNK, std::max<uint32_t>(ri.n_rows, 1u));
    const uint32_t forced_sub = rs_env("FXHIP_RS_SUB_ROWS"), forced_chunk = rs_env("FXHIP_RS_CHUNK_ROWS");
    uint32_t best_sub = 0, best_cr = 0, best_n = 0;
    bool best_side = false, best_lean = false;
    int best_per_cu = 0;
    // The kernel built for five loads per lane and sub-tile first (fewer registers), the one for six
    // where it saves a sub-tile per chunk; with the chunk's table of side values in LDS, and without
    // it where the table would cost a workgroup per CU or a sub-tile per chunk (the rows then load
    // their side values themselves).  Fewest sub-tiles per chunk wins, the first found among equals.
    const uint32_t forced_loads = rs_env("FXHIP_RS_LOADS");   // tuning aid: FX_RS_KV or FX_RS_KV_LEAN
    // (a launch with more chunks than the device holds workgroups runs the build with persistent
    // workgroups, which exists for six loads only)
    // (and a map whose tables are uploaded runs the build that reads them from device memory:
    // persistent workgroups as well, a map of that many tasks seldom fits the device)
    const bool beyond = pl->wide || (uint64_t)((ri.n_rows + FX_BLOCK - 1) / FX_BLOCK) * ri.n_tasks > (uint64_t)std::max(cus, 1) * FX_RS_OCC;
    for (int lean = beyond ? 0 : 1; lean >= 0; --lean) {
      const void* fn = pl->wide ? kern->fn_wide : beyond ? kern->fn_persist : lean ? kern->fn_lean : kern->fn;
      if (!fn || (forced_loads && forced_loads != (lean ? FX_RS_KV_LEAN : FX_RS_KV))) continue;
      // (measured on the benchmark's shape: 22.6 against 22.95 us for kernels that store as they
      // compute; with outputs staged in LDS, where LDS and not registers bounds the occupancy, 25.6 against 24.4)
      if (lean && kern->n_staged != 0 && !forced_loads) continue;
      const uint32_t max_sub = rs_max_sub_rows(ri, lean ? FX_RS_KV_LEAN : FX_RS_KV);
      if (max_sub < 8u) continue;
      for (int with_side = kern->side_row_words != 0 ? 1 : 0; with_side >= 0; --with_side) {
        for (uint32_t sub = max_sub; sub >= 8u; sub = sub > 8u ? std::max<uint32_t>(8u, sub - 4u) : 0u) {
          if (forced_sub && sub > forced_sub) continue;
          // at most the occupancy the kernels are compiled for: a launch that needs a seventh slot per CU
          // is not placed at once and takes 27.4 us where six per CU take 23.4 us
          auto slots = [&](uint32_t chunk_rows) {
            int n = 0;
            if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, fn, (int)FX_BLOCK,
                                                             (size_t)rs_lds_bytes(ri, kern, sub, chunk_rows, with_side != 0)) != hipSuccess) {
              (void)hipGetLastError();
              return 0;
            }
            return std::min(n, (int)FX_RS_OCC);
          };
          auto chunkFor = [&](int per_cu) {
            const uint32_t resident = (uint32_t)per_cu * (uint32_t)std::max(cus, 1);
            const uint32_t per_task = std::max<uint32_t>(1u, resident / std::max<uint32_t>(ri.n_tasks, 1u));
            uint32_t c = (ri.n_rows + per_task - 1) / per_task;
            c = std::min<uint32_t>(FX_BLOCK, std::max<uint32_t>(c, min_chunk));
            if (forced_chunk) c = std::min<uint32_t>(FX_BLOCK, std::max<uint32_t>(forced_chunk, min_chunk));
            return c;
          };
          // the table is part of the LDS, and the chunk follows from the number of resident
          // workgroups: from the largest chunk down until both agree
          int per_cu = slots(FX_BLOCK);
          if (per_cu < 1) continue;
          uint32_t cr = chunkFor(per_cu);
          for (int round = 0; round < 3; ++round) {
            const int better = slots(cr);
            if (better <= per_cu) break;
            per_cu = better;
            cr = chunkFor(per_cu);
          }
          const uint32_t n = (cr + sub - 1) / sub;
          if (rs_env("FXHIP_RS_VERBOSE"))
            fprintf(stderr, "[fxhip] row-stream geometry: %u loads, side table %d, sub-tile %u rows, %u B of LDS, %d workgroups per CU, chunk %u rows, %u sub-tiles\n",
                    lean ? FX_RS_KV_LEAN : FX_RS_KV, with_side, sub, rs_lds_bytes(ri, kern, sub, cr, with_side != 0), per_cu, cr, n);
          if (best_sub == 0 || n < best_n) { best_sub = sub; best_cr = cr; best_n = n; best_side = with_side != 0; best_lean = lean != 0; best_per_cu = per_cu; }
          if (forced_sub || sub == 8u) break;
        }
      }
    }
    if (best_sub == 0) return fail(FX_E_LIMIT, "row-stream kernel: no sub-tile size fits the device");
    pl->rs_sub_rows = best_sub;
    pl->rs_chunk_rows = best_cr;
    pl->rs_side_lds = best_side ? 1u : 0u;
    pl->rs_lean = best_lean ? 1u : 0u;
    pl->rs_grid_cap = (uint32_t)best_per_cu * (uint32_t)std::max(cus, 1);   // workgroups that the device holds at once
  }
  rl->sub_rows = pl->rs_sub_rows;
  rl->chunk_rows = pl->rs_chunk_rows;
  rl->side_lds = pl->rs_side_lds;
  rl->chunks = (ri.n_rows + rl->chunk_rows - 1) / rl->chunk_rows;
  fx_rs_finish_geometry(rl);
  const uint32_t cr = rl->chunk_rows;
  // A launch whose first sub-tiles alone are megabytes of requests floods the memory system: there
  // the counts get a head start.  A small launch would only lose the time.
  const uint64_t first_bytes = (uint64_t)rl->chunks * ri.n_tasks * std::min<uint32_t>(cr, rl->sub_rows) * ri.S * 4u;
  rl->bulk_delay = first_bytes >= FX_RS_FLOOD_BYTES ? FX_RS_BULK_DELAY : 0u;
  if (const uint32_t d = rs_env("FXHIP_RS_BULK_DELAY")) rl->bulk_delay = d - 1u;   // tuning aids (value + 1; FXHIP_RS_LATE_TELL=1)
  rl->late_tell = rs_env("FXHIP_RS_LATE_TELL") ? 1u : 0u;
  return FX_OK;
}
// (persistent workgroups: at most as many as the device holds at once, each takes chunks in turn)
static hipError_t rs_launch(const FxRsKernel* kern, const FxRsInfo& ri, const FxRsLaunch& rl, const FxDyn* dyn, hipStream_t stream,
                            bool lean, uint32_t grid_cap) {
  const uint32_t n_chunks = rl.chunks * rl.n_tasks, cap = std::max<uint32_t>(grid_cap, 1u);
  if (n_chunks == 0) return hipSuccess;
  const bool persist = n_chunks > cap;
  const uint32_t grid = persist ? cap : n_chunks;
  void* args[2] = {(void*)&rl, (void*)dyn};
  if (rl.wide != 0 && !kern->fn_wide) return hipErrorInvalidDeviceFunction;   // (rs_of has looked)
  return hipLaunchKernel(rl.wide != 0 ? kern->fn_wide : persist ? kern->fn_persist : (lean && kern->fn_lean ? kern->fn_lean : kern->fn), dim3(grid), dim3(FX_BLOCK), args, rs_lds_bytes(ri, kern, rl.sub_rows, rl.chunk_rows, rl.side_lds != 0), stream);
}

// ---- class-map head kernel (fx_cmap.h): geometry of a launch ----
#define FX_CMAP_EPOCH_MAX 0xffffu   // the epoch tag of its 64-bit status words has 16 bits
static size_t cmap_status_words(const FxCmapInfo& ci) {
  const uint32_t chunks = (ci.n_rows + fx_cmap_chunk_rows() - 1) / fx_cmap_chunk_rows();
  return (size_t)chunks * ((ci.n_tasks + 7u) / 8u) * 2u;
}
// One workgroup per chunk of rows; the kernel is chosen only when the device holds all of them
// at once (a workgroup waits for the counts of the chunks before its own).
static int cmap_launch_info(fx::Plan* pl, FxCmapLaunch* hl, bool* fits, bool* wide) {
  const FxCmapInfo& ci = pl->cmap;
  memset(hl, 0, sizeof(*hl));
  hl->n_rows = ci.n_rows;
  hl->n_tasks = ci.n_tasks;
  hl->chunk_rows = fx_cmap_chunk_rows();
  hl->chunks = (ci.n_rows + hl->chunk_rows - 1) / hl->chunk_rows;
  hl->C = ci.C;
  hl->first = ci.first;
  hl->thr_bits = ci.thr_bits;
  hl->var_xy_bits = ci.var_xy_bits;
  hl->var_wh_bits = ci.var_wh_bits;
  hl->spin_limit = g_stream_spin.load(std::memory_order_relaxed);
  hl->n_sptr = (uint32_t)pl->sptr.size();
  hl->n_tptr = (uint32_t)pl->tptr.size();
  hl->conf_slot = ci.conf_slot;
  hl->loc_slot = ci.loc_slot;
  hl->pri_slot = ci.pri_slot;
  for (int k = 0; k < 2; ++k) {
    hl->out_slot[k] = ci.out_slot[k];
    hl->out_tstride[k] = ci.out_tstride[k];
  }
  if (pl->head_resident == 0) {
    uint32_t w = 0, n = 0;
    HIP_OK(fx_cmap_resident(fx_cmap_lds_bytes(*hl), &w, &n));
    pl->cmap_resident_wide = w;
    pl->head_resident = std::max<uint32_t>(n, 1u);
  }
  *wide = hl->chunks <= pl->cmap_resident_wide;
  *fits = *wide || hl->chunks <= pl->head_resident;
  return FX_OK;
}

static int upload_blob(fx_region* reg, fx::Plan* pl, int dev) {
  std::lock_guard<std::mutex> g(reg->mu);
  if (!pl->dev_blob || pl->dev_id != dev) {
    void* d = nullptr;
    HIP_OK(hipMalloc(&d, pl->blob.size() * 4));
    HIP_OK(hipMemcpy(d, pl->blob.data(), pl->blob.size() * 4, hipMemcpyHostToDevice));
    pl->dev_blob = d;
    pl->dev_id = dev;
  }
  return FX_OK;
}

static int run_impl(fx_region* reg, const fx_plan* plan, const fx_arg* args, int n_args, void* const* out_ptrs,
                    void* scratch, uint32_t* totals_host, void* stream_, float* kernel_ms, int cap, int* n_kernels,
                    int repeat = 1) {
  if (!reg || !plan || !out_ptrs) return fail(FX_E_INVALID, "null argument");
  fx::Plan* pl = const_cast<fx::Plan*>(P(plan));
  if (pl->region != &reg->r) return fail(FX_E_INVALID, "plan does not belong to this region");
  if (n_args != pl->n_args) return fail(FX_E_INVALID, "argument count differs from the plan");
  if (pl->mode == FX_MODE_COMPACT && (!scratch || !totals_host))
    return fail(FX_E_INVALID, "compacting region needs scratch memory and a pinned totals buffer");
  hipStream_t stream = (hipStream_t)stream_;

  int dev = 0;
  HIP_OK(hipGetDevice(&dev));
  int rc = upload_blob(reg, pl, dev);
  if (rc != FX_OK) return rc;
  const FxSpecKernels* spec = spec_of(pl);
  if (!spec && pl->needs_compiled) {
    char key[17];
    snprintf(key, sizeof key, "%016llx", (unsigned long long)pl->spec_key);
    return fail(FX_E_LIMIT, std::string("the interpreter's temporaries of this region need ") + std::to_string(pl->lds_bytes) +
                                " bytes of LDS (limit 162816) and no compiled kernels for its programs (key " + key +
                                ") are linked in or enabled: generate them with fx_plan_spec_source / python -m functs_amd.aot");
  }
  FxLaunchInfo li = launch_info(pl);
  // The one-launch forms tag their status words with the call's epoch, which travels in the
  // kernel arguments: a captured launch would be replayed with the epoch of the capture and read
  // the counts of an earlier replay.  Under stream capture the two-pass form is recorded instead.
  hipStreamCaptureStatus cap_status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &cap_status) != hipSuccess) {
    (void)hipGetLastError();
    cap_status = hipStreamCaptureStatusNone;
  }
  const bool capturing = cap_status != hipStreamCaptureStatusNone;
  void* status = nullptr;
  uint32_t epoch = 0;
  const FxRsKernel* rsk = capturing ? nullptr : rs_of(pl);
  FxRsLaunch rl;
  if (rsk) {
    rc = rs_launch_info(pl, rsk, &rl);
    if (rc != FX_OK) return rc;
    void* rstatus = nullptr;
    rc = status_words(reg, pl->head_status, rs_status_words(pl->rs), stream, dev, &rstatus, &epoch, repeat);
    if (rc != FX_OK) return rc;
    if (!rstatus) rsk = nullptr;
    rl.status = (uint32_t*)rstatus;
    rl.totals = totals_host;
  }
  bool head = !rsk && !capturing && head_fits(pl);
  FxHeadLaunch hl;
  if (head) {
    rc = head_launch_info(pl, &hl);
    if (rc != FX_OK) return rc;
    void* hstatus = nullptr;
    rc = status_words(reg, pl->head_status, head_status_words(pl->head), stream, dev, &hstatus, &epoch, repeat);
    if (rc != FX_OK) return rc;
    if (!hstatus) head = false;
    hl.status = (uint32_t*)hstatus;
    hl.totals = totals_host;
  }
  bool cmap = !rsk && !head && !capturing && cmap_active(pl), cmap_wide = false;
  FxCmapLaunch cl;
  if (cmap) {
    rc = cmap_launch_info(pl, &cl, &cmap, &cmap_wide);
    if (rc != FX_OK) return rc;
  }
  if (cmap) {
    void* cstatus = nullptr;
    rc = status_words(reg, pl->head_status, cmap_status_words(pl->cmap), stream, dev, &cstatus, &epoch, repeat, FX_CMAP_EPOCH_MAX);
    if (rc != FX_OK) return rc;
    if (!cstatus) cmap = false;
    cl.status = (uint32_t*)cstatus;
    cl.totals = totals_host;
  }
  bool streaming = !rsk && !head && !cmap && !capturing && pl->mode == FX_MODE_COMPACT && stream_active(pl, spec);
  if (streaming) {
    rc = stream_status(reg, pl, stream, dev, &status, &epoch, repeat);
    if (rc != FX_OK) return rc;
    if (!status) streaming = false;
  }
  FxDyn dyn;
  if (pl->wide) {
    // a map of many tasks: the tables go to the end of the caller's scratch memory, in stream
    // order ahead of the kernels that stage them from there
    if (!scratch) return fail(FX_E_INVALID, "this plan keeps its tables in scratch memory (fx_plan_scratch_bytes): scratch is null");
    std::vector<uint64_t> words(pl->wide_bytes / 8, 0);
    rc = fill_tables(pl, args, out_ptrs, scratch, totals_host, pl->dev_blob, words.data(), (uint32_t*)(words.data() + li.n_p), status);
    if (rc != FX_OK) return rc;
    void* table = (char*)scratch + pl->wide_off;
    HIP_OK(fx_upload_words(words.data(), (size_t)li.n_p + ((size_t)li.n_s + 1) / 2, table, stream));
    li.wide = (uint64_t)(uintptr_t)table;
    rl.wide = li.wide;
    memset(&dyn, 0, sizeof dyn);
  } else {
    rc = fill_dyn(pl, args, out_ptrs, scratch, totals_host, pl->dev_blob, &dyn, status);
    if (rc != FX_OK) return rc;
  }
  const uint32_t* sb = (const uint32_t*)pl->dev_blob;
  if (pl->mode == FX_MODE_COMPACT) {
    // Tasks without rows launch no tile: their total is published here.  The others hold a
    // mark until the last tile of the task stores the count (fx_region_wait_totals looks for
    // it).  The caller must not reuse totals_host while an earlier run is still in flight.
    for (int t = 0; t < reg->r.degree; ++t)
      totals_host[t] = (pl->out_shape.empty() || pl->out_shape[0][t].empty() || pl->out_shape[0][t][0] > 0)
                           ? FX_TOTAL_PENDING
                           : 0u;
  }
  const int launches = rsk ? (rl.chunks * rl.n_tasks > 0 ? 1 : 0) : head ? (hl.chunks * hl.n_tasks > 0 ? 1 : 0) : cmap ? (cl.chunks > 0 ? 1 : 0) : streaming ? (pl->stream.grid > 0 ? 1 : 0) : pl->launches;
  g_launches.fetch_add((uint64_t)launches, std::memory_order_relaxed);
  if (spec || rsk || head || cmap) g_spec_launches.fetch_add((uint64_t)launches, std::memory_order_relaxed);
  // optional per-kernel timing with events on the launch stream
  hipEvent_t ev[4] = {nullptr, nullptr, nullptr, nullptr};
  const bool timed = kernel_ms != nullptr;
  int nk = 0;
  if (timed)
    for (auto& e : ev) HIP_OK(hipEventCreate(&e));
  auto mark = [&](int i) -> hipError_t { return timed ? hipEventRecord(ev[i], stream) : hipSuccess; };
  if (pl->mode == FX_MODE_DENSE) {
    HIP_OK(mark(0));
    // persistent workgroups: at most FX_DENSE_WG_PER_CU per CU worth of blocks stride over the units
    for (int r = 0; r < repeat; ++r)
      HIP_OK(fx_launch_dense(pl->max_rank, sb, li, &dyn, std::min<uint32_t>(pl->grid, 256u * FX_DENSE_WG_PER_CU), stream, spec, lean_of(pl), pl->lean_slot_err));
    HIP_OK(mark(1));
    nk = pl->grid > 0 ? 1 : 0;
  } else if (rsk) {
    HIP_OK(mark(0));
    for (int r = 0; r < repeat; ++r) {
      rl.epoch = epoch + (uint32_t)r;
      HIP_OK(rs_launch(rsk, pl->rs, rl, &dyn, stream, pl->rs_lean != 0, pl->rs_grid_cap));
    }
    HIP_OK(mark(1));
    nk = rl.chunks * rl.n_tasks > 0 ? 1 : 0;
  } else if (head) {
    HIP_OK(mark(0));
    for (int r = 0; r < repeat; ++r) {
      hl.epoch = epoch + (uint32_t)r;
      HIP_OK(fx_launch_head_stream(hl, &dyn, stream));
    }
    HIP_OK(mark(1));
    nk = hl.chunks * hl.n_tasks > 0 ? 1 : 0;
  } else if (cmap) {
    HIP_OK(mark(0));
    for (int r = 0; r < repeat; ++r) {
      cl.epoch = epoch + (uint32_t)r;
      HIP_OK(fx_launch_classmap_head(cl, &dyn, cmap_wide, stream));
    }
    HIP_OK(mark(1));
    nk = cl.chunks > 0 ? 1 : 0;
  } else if (streaming) {
    HIP_OK(mark(0));
    for (int r = 0; r < repeat; ++r) {
      li.epoch = epoch + (uint32_t)r;
      li.total_units = pl->stream.grid;
      HIP_OK(fx_launch_compact_stream(pl->max_rank, sb, li, &dyn, stream_grid(pl), stream, spec));
    }
    HIP_OK(mark(1));
    nk = pl->stream.grid > 0 ? 1 : 0;
  } else {
    HIP_OK(mark(0));
    for (int r = 0; r < repeat; ++r) HIP_OK(fx_launch_compact_count(sb, li, &dyn, pl->grid_count, stream, spec));
    HIP_OK(mark(1));
    HIP_OK(mark(2));
    for (int r = 0; r < repeat; ++r) HIP_OK(fx_launch_compact_scatter(pl->max_rank, sb, li, &dyn, pl->grid, stream, spec));
    HIP_OK(mark(3));
    nk = pl->grid > 0 ? 2 : 0;
  }
  if (timed) {
    HIP_OK(hipEventSynchronize(ev[nk == 2 ? 3 : 1]));
    for (int k = 0; k < nk && k < cap; ++k) {
      HIP_OK(hipEventElapsedTime(&kernel_ms[k], ev[2 * k], ev[2 * k + 1]));
      kernel_ms[k] /= (float)repeat;
    }
    for (auto& e : ev) (void)hipEventDestroy(e);
    if (n_kernels) *n_kernels = nk;
  }
  return FX_OK;
}

// Launches over several argument sets of one plan in rotation, inside ONE event pair:
// `which` < 0 launches every kernel of the call in order (a whole call per set), otherwise only
// kernel `which` of the call (the others must have run on every set before: a kernel of a
// compacting region reads what the count pass of its own set left in that set's scratch).
// With sets that together exceed the last-level cache every launch works on cold lines.
int fx_region_run_timed_sets(fx_region* reg, const fx_plan* plan, int n_sets, const fx_arg* const* args, int n_args,
                             void* const* const* out_ptrs, void* const* scratch, uint32_t* const* totals_host,
                             void* stream_, int which, int rounds, float* ms_mean) {
  if (!reg || !plan || !args || !out_ptrs || !ms_mean) return fail(FX_E_INVALID, "null argument");
  if (n_sets < 1 || n_sets > 64 || rounds < 1 || rounds > 1000)
    return fail(FX_E_INVALID, "fx_region_run_timed_sets: 1..64 sets, 1..1000 rounds");
  fx::Plan* pl = const_cast<fx::Plan*>(P(plan));
  if (pl->region != &reg->r) return fail(FX_E_INVALID, "plan does not belong to this region");
  if (n_args != pl->n_args) return fail(FX_E_INVALID, "argument count differs from the plan");
  const bool compact = pl->mode == FX_MODE_COMPACT;
  if (compact && (!scratch || !totals_host)) return fail(FX_E_INVALID, "compacting region needs scratch and totals per set");
  // (a plan whose tables are uploaded keeps them in every set's scratch memory, dense or not)
  const bool with_scratch = compact || pl->wide;
  if (pl->wide && !scratch) return fail(FX_E_INVALID, "this plan keeps its tables in scratch memory (fx_plan_scratch_bytes): scratch per set");
  hipStream_t stream = (hipStream_t)stream_;
  // one untimed call per set: uploads the descriptor, leaves every set's scratch valid
  for (int i = 0; i < n_sets; ++i) {
    const int rc = run_impl(reg, plan, args[i], n_args, out_ptrs[i], with_scratch ? scratch[i] : nullptr,
                            compact ? totals_host[i] : nullptr, stream_, nullptr, 0, nullptr);
    if (rc != FX_OK) return rc;
  }
  const FxSpecKernels* spec = spec_of(pl);
  FxLaunchInfo li = launch_info(pl);
  void* status = nullptr;
  uint32_t epoch = 0;
  int dev = 0;
  HIP_OK(hipGetDevice(&dev));
  const FxRsKernel* rsk = compact ? rs_of(pl) : nullptr;
  FxRsLaunch rl;
  if (rsk) {
    int rc = rs_launch_info(pl, rsk, &rl);
    if (rc != FX_OK) return rc;
    void* rstatus = nullptr;
    rc = status_words(reg, pl->head_status, rs_status_words(pl->rs), stream, dev, &rstatus, &epoch, rounds * n_sets);
    if (rc != FX_OK) return rc;
    if (!rstatus) rsk = nullptr;
    rl.status = (uint32_t*)rstatus;
  }
  bool head = !rsk && compact && head_fits(pl);
  FxHeadLaunch hl;
  if (head) {
    int rc = head_launch_info(pl, &hl);
    if (rc != FX_OK) return rc;
    void* hstatus = nullptr;
    rc = status_words(reg, pl->head_status, head_status_words(pl->head), stream, dev, &hstatus, &epoch, rounds * n_sets);
    if (rc != FX_OK) return rc;
    if (!hstatus) head = false;
    hl.status = (uint32_t*)hstatus;
  }
  bool cmap = !rsk && !head && compact && cmap_active(pl), cmap_wide = false;
  FxCmapLaunch cl;
  if (cmap) {
    int rc = cmap_launch_info(pl, &cl, &cmap, &cmap_wide);
    if (rc != FX_OK) return rc;
  }
  if (cmap) {
    if ((uint32_t)(rounds * n_sets) >= FX_CMAP_EPOCH_MAX)
      return fail(FX_E_INVALID, "fx_region_run_timed_sets: at most 65534 launches of this kernel in one call");
    void* cstatus = nullptr;
    const int rc = status_words(reg, pl->head_status, cmap_status_words(pl->cmap), stream, dev, &cstatus, &epoch, rounds * n_sets,
                                FX_CMAP_EPOCH_MAX);
    if (rc != FX_OK) return rc;
    if (!cstatus) cmap = false;
    cl.status = (uint32_t*)cstatus;
  }
  bool streaming = !rsk && !head && !cmap && compact && stream_active(pl, spec);
  if (streaming) {
    const int rc = stream_status(reg, pl, stream, dev, &status, &epoch, rounds * n_sets);
    if (rc != FX_OK) return rc;
    if (!status) streaming = false;
  }
  if (which >= ((streaming || rsk || head || cmap) ? 1 : pl->launches)) return fail(FX_E_INVALID, "fx_region_run_timed_sets: the call has no such kernel");
  std::vector<FxDyn> dyn((size_t)n_sets);
  for (int i = 0; i < n_sets; ++i) {
    memset(&dyn[i], 0, sizeof(FxDyn));
    if (pl->wide) continue;   // (the untimed call above has left the set's tables in its scratch memory)
    const int rc = fill_dyn(pl, args[i], out_ptrs[i], compact ? scratch[i] : nullptr, compact ? totals_host[i] : nullptr,
                            pl->dev_blob, &dyn[i], status);
    if (rc != FX_OK) return rc;
  }
  const uint32_t* sb = (const uint32_t*)pl->dev_blob;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  HIP_OK(hipEventCreate(&e0));
  HIP_OK(hipEventCreate(&e1));
  HIP_OK(hipStreamSynchronize(stream));
  HIP_OK(hipEventRecord(e0, stream));
  for (int r = 0; r < rounds; ++r)
    for (int i = 0; i < n_sets; ++i) {
      if (pl->wide) {
        li.wide = (uint64_t)(uintptr_t)((char*)scratch[i] + pl->wide_off);
        rl.wide = li.wide;
      }
      if (!compact) {
        HIP_OK(fx_launch_dense(pl->max_rank, sb, li, &dyn[i], std::min<uint32_t>(pl->grid, 256u * FX_DENSE_WG_PER_CU), stream, spec, lean_of(pl), pl->lean_slot_err));
      } else if (rsk) {
        rl.epoch = epoch + (uint32_t)(r * n_sets + i);
        rl.totals = totals_host[i];
        HIP_OK(rs_launch(rsk, pl->rs, rl, &dyn[i], stream, pl->rs_lean != 0, pl->rs_grid_cap));
      } else if (head) {
        hl.epoch = epoch + (uint32_t)(r * n_sets + i);
        hl.totals = totals_host[i];
        HIP_OK(fx_launch_head_stream(hl, &dyn[i], stream));
      } else if (cmap) {
        cl.epoch = epoch + (uint32_t)(r * n_sets + i);
        cl.totals = totals_host[i];
        HIP_OK(fx_launch_classmap_head(cl, &dyn[i], cmap_wide, stream));
      } else if (streaming) {
        li.epoch = epoch + (uint32_t)(r * n_sets + i);
        li.total_units = pl->stream.grid;
        HIP_OK(fx_launch_compact_stream(pl->max_rank, sb, li, &dyn[i], stream_grid(pl), stream, spec));
      } else {
        if (which < 0 || which == 0) HIP_OK(fx_launch_compact_count(sb, li, &dyn[i], pl->grid_count, stream, spec));
        if (which < 0 || which == 1) HIP_OK(fx_launch_compact_scatter(pl->max_rank, sb, li, &dyn[i], pl->grid, stream, spec));
      }
    }
  HIP_OK(hipEventRecord(e1, stream));
  HIP_OK(hipEventSynchronize(e1));
  float ms = 0.f;
  HIP_OK(hipEventElapsedTime(&ms, e0, e1));
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  *ms_mean = ms / (float)(rounds * n_sets);
  return FX_OK;
}

int fx_region_poll_totals(const fx_plan* plan, const uint32_t* totals_host, uint32_t spin_us) {
  if (!plan || !totals_host) return fail(FX_E_INVALID, "null argument");
  const fx::Plan* pl = P(plan);
  if (pl->mode != FX_MODE_COMPACT) return fail(FX_E_INVALID, "not a compacting region");
  const volatile uint32_t* tot = totals_host;
  const int T = pl->region->degree;
  using clock = std::chrono::steady_clock;
  const clock::time_point t0 = clock::now();
  const clock::duration budget = std::chrono::microseconds(spin_us);
  for (;;) {
    bool all = true;
    for (int t = 0; t < T; ++t) all = all && tot[t] != FX_TOTAL_PENDING;
    if (all) {
      std::atomic_thread_fence(std::memory_order_acquire);
      return 1;
    }
    if (clock::now() - t0 >= budget) return 0;
    __builtin_ia32_pause();
  }
}

int fx_region_wait_totals(const fx_plan* plan, const uint32_t* totals_host, void* stream_) {
  if (!plan || !totals_host) return fail(FX_E_INVALID, "null argument");
  const fx::Plan* pl = P(plan);
  if (pl->mode != FX_MODE_COMPACT) return fail(FX_E_INVALID, "not a compacting region");
  hipStream_t stream = (hipStream_t)stream_;
  const volatile uint32_t* tot = totals_host;
  const int T = pl->region->degree;
  // The count of a task is stored by its last tile early in the second pass, through
  // host-coherent memory: it is usually here well before the kernel has finished, and the
  // host looks for it from its own core.  Counts that take longer than the polling budget
  // (a stream with other work queued ahead of the launch, memory that the host does not see
  // until the stream has drained) are waited for in the runtime's stream synchronisation,
  // which does not keep a core busy for that long.
  using clock = std::chrono::steady_clock;
  const clock::time_point t0 = clock::now();
  const clock::duration budget = std::chrono::microseconds(g_totals_spin_us.load(std::memory_order_relaxed));
  clock::time_point next_query = t0 + std::chrono::microseconds(50);
  for (;;) {
    bool all = true;
    for (int t = 0; t < T; ++t) all = all && tot[t] != FX_TOTAL_PENDING;
    if (all) {
      std::atomic_thread_fence(std::memory_order_acquire);
      return FX_OK;
    }
    const clock::time_point now = clock::now();
    if (now - t0 >= budget) break;
    __builtin_ia32_pause();
    if (now >= next_query) {
      // the runtime is asked rarely: a query takes its locks and slows the launches of other threads
      const hipError_t q = hipStreamQuery(stream);
      if (q == hipSuccess) break;
      if (q != hipErrorNotReady) HIP_OK(q);
      next_query = now + std::chrono::microseconds(50);
    }
  }
  HIP_OK(hipStreamSynchronize(stream));
  for (int t = 0; t < T; ++t)
    if (tot[t] == FX_TOTAL_PENDING) return fail(FX_E_HIP, "a task's kept-row count was never written");
  return FX_OK;
}

int fx_region_run(fx_region* reg, const fx_plan* plan, const fx_arg* args, int n_args, void* const* out_ptrs,
                  void* scratch, uint32_t* totals_host, void* stream) {
  return run_impl(reg, plan, args, n_args, out_ptrs, scratch, totals_host, stream, nullptr, 0, nullptr);
}

int fx_region_run_timed(fx_region* reg, const fx_plan* plan, const fx_arg* args, int n_args, void* const* out_ptrs,
                        void* scratch, uint32_t* totals_host, void* stream, float* kernel_ms, int cap,
                        int* n_kernels) {
  if (!kernel_ms || cap < 2) return fail(FX_E_INVALID, "fx_region_run_timed: kernel_ms[>=2] required");
  return run_impl(reg, plan, args, n_args, out_ptrs, scratch, totals_host, stream, kernel_ms, cap, n_kernels);
}

int fx_region_run_timed_batched(fx_region* reg, const fx_plan* plan, const fx_arg* args, int n_args,
                                void* const* out_ptrs, void* scratch, uint32_t* totals_host, void* stream, int repeat,
                                float* kernel_ms, int cap, int* n_kernels) {
  if (!kernel_ms || cap < 2) return fail(FX_E_INVALID, "fx_region_run_timed_batched: kernel_ms[>=2] required");
  if (repeat < 1 || repeat > 1000) return fail(FX_E_INVALID, "fx_region_run_timed_batched: repeat must be 1..1000");
  return run_impl(reg, plan, args, n_args, out_ptrs, scratch, totals_host, stream, kernel_ms, cap, n_kernels, repeat);
}

size_t fx_compact_rows_scratch_bytes(int64_t n) {
  if (n < 0) n = 0;
  return (size_t)(((n + FX_BLOCK - 1) / FX_BLOCK + 1) * 4 + 256);
}

static_assert(FX_STATIC_MAX_ROWS == FX_COMPACT_ROWS_STATIC_MAX, "the header states the limit of the static array");
// argument checks shared by fx_compact_rows and fx_compact_rows_static
static int check_compact_rows(const uint8_t* mask, int64_t n, const void* const* cols, void* const* outs,
                              const int32_t* rowlen, const int32_t* elsize, int n_cols, const uint32_t* total_host) {
  if (n < 0 || n_cols < 0 || n_cols > 8) return fail(FX_E_INVALID, "fx_compact_rows: n >= 0 and 0 <= n_cols <= 8");
  if (n >= ((int64_t)1 << 31)) return fail(FX_E_LIMIT, "fx_compact_rows: n above 2^31");
  if (!total_host) return fail(FX_E_INVALID, "fx_compact_rows: total_host is required");
  if (n > 0 && !mask) return fail(FX_E_INVALID, "fx_compact_rows: null mask");
  for (int i = 0; i < n_cols; ++i) {
    if (!cols || !outs || !rowlen || !elsize) return fail(FX_E_INVALID, "fx_compact_rows: null column arrays");
    if (elsize[i] != 4 && elsize[i] != 8 && elsize[i] != 1) return fail(FX_E_UNSUPPORTED, "fx_compact_rows: elsize 1, 4 or 8");
    if (rowlen[i] < 1) return fail(FX_E_INVALID, "fx_compact_rows: rowlen >= 1");
    if ((int64_t)rowlen[i] * n >= ((int64_t)1 << 31)) return fail(FX_E_LIMIT, "fx_compact_rows: column above 2^31 elements");
  }
  return FX_OK;
}

int fx_compact_rows_static(const uint8_t* mask, int64_t n, const void* const* cols, void* const* outs,
                           const int32_t* rowlen, const int32_t* elsize, int n_cols, uint32_t* total_host,
                           void* stream_) {
  const int rc = check_compact_rows(mask, n, cols, outs, rowlen, elsize, n_cols, total_host);
  if (rc != FX_OK) return rc;
  if (n > FX_STATIC_MAX_ROWS)
    return fail(FX_E_LIMIT, "fx_compact_rows_static: n = " + std::to_string(n) + " rows is above the limit of " +
                                std::to_string((long long)FX_STATIC_MAX_ROWS) + " (FX_COMPACT_ROWS_STATIC_MAX); use fx_compact_rows with caller scratch");
  if (n == 0) {
    *total_host = 0;
    return FX_OK;
  }
  HIP_OK(fx_launch_compact_rows_static(mask, n, cols, outs, rowlen, elsize, n_cols, total_host, (hipStream_t)stream_));
  return FX_OK;
}

int fx_compact_rows(const uint8_t* mask, int64_t n, const void* const* cols, void* const* outs, const int32_t* rowlen,
                    const int32_t* elsize, int n_cols, void* scratch, size_t scratch_bytes, uint32_t* total_host,
                    void* stream_) {
  const int rc = check_compact_rows(mask, n, cols, outs, rowlen, elsize, n_cols, total_host);
  if (rc != FX_OK) return rc;
  if (n > 0 && !scratch) return fail(FX_E_INVALID, "fx_compact_rows: null mask/scratch");
  if (scratch_bytes < fx_compact_rows_scratch_bytes(n)) return fail(FX_E_INVALID, "fx_compact_rows: scratch too small");
  if (n == 0) {
    *total_host = 0;
    return FX_OK;
  }
  HIP_OK(fx_launch_compact_rows(mask, n, cols, outs, rowlen, elsize, n_cols, (uint32_t*)scratch, total_host,
                                (hipStream_t)stream_));
  return FX_OK;
}

// ---- stacked LSTM recurrence as one persistent kernel (fx_lstm.hip) ----
int fx_lstm_stack_fits(int batch, int hidden, int layers) {
  if (hidden < 32 || hidden > 1024 || (hidden & (hidden - 1)) != 0) return 0;
  if (layers < 1 || layers > 4 || batch < 1 || batch > 16) return 0;
  // 1024 hidden units are resident together only at four waves per SIMD, 128 registers a lane, of
  // which the weight columns may take 64 (at 512 and below every L fits)
  if (hidden == 1024 && layers * (hidden / 32) > 64) return 0;
  return 1;
}
size_t fx_lstm_stack_workspace_bytes(int batch, int hidden, int layers) {
  if (batch < 1 || hidden < 1 || layers < 1) return 0;
  return (size_t)FX_LSTM_CTL_WORDS * 4 + (size_t)2 * layers * batch * hidden * 8;
}

int fx_lstm_stack(const float* x, const float* wih, const float* whh, const float* bih, const float* bhh, const float* h0,
                  const float* c0, float* out, float* state_h, float* state_c, int seq_len, int batch, int hidden,
                  int layers, void* workspace, size_t workspace_bytes, void* stream_) {
  if (!x || !wih || !whh || !bih || !bhh || !out || !state_h || !state_c || !workspace)
    return fail(FX_E_INVALID, "fx_lstm_stack: null argument");   // h0 / c0 may be null: zero initial state
  if (seq_len < 1 || batch < 1 || hidden < 1 || layers < 1) return fail(FX_E_INVALID, "fx_lstm_stack: sizes must be positive");
  if (workspace_bytes < fx_lstm_stack_workspace_bytes(batch, hidden, layers))
    return fail(FX_E_INVALID, "fx_lstm_stack: workspace smaller than fx_lstm_stack_workspace_bytes");
  if (((uintptr_t)workspace & 255u) != 0) return fail(FX_E_INVALID, "fx_lstm_stack: workspace must be 256-byte aligned");
  if (!fx_lstm_stack_fits(batch, hidden, layers))
    return fail(FX_E_UNSUPPORTED, "fx_lstm_stack: hidden must be a power of two in 32..1024, 1..4 layers (2 at hidden 1024), batch up to 16 (got hidden " +
                                      std::to_string(hidden) + ", layers " + std::to_string(layers) + ", batch " + std::to_string(batch) + ")");
  FxLstmArgs a;
  a.x = x; a.wih = wih; a.whh = whh; a.bih = bih; a.bhh = bhh; a.h0 = h0; a.c0 = c0;
  a.out = out; a.state_h = state_h; a.state_c = state_c;
  a.ctl = (uint32_t*)workspace;
  a.hbuf = (uint64_t*)((char*)workspace + (size_t)FX_LSTM_CTL_WORDS * 4);
  a.err_host = err_word(true);
  a.T = seq_len; a.B = batch; a.H = hidden;
  a.spin_limit = g_lstm_spin.load(std::memory_order_relaxed);
  const int rc = fx_launch_lstm_stack(a, layers, (hipStream_t)stream_);
  if (rc == 1) return fail(FX_E_UNSUPPORTED, "fx_lstm_stack: no kernel for these sizes");
  if (rc == 2)
    return fail(FX_E_LIMIT, "fx_lstm_stack: " + std::to_string(hidden / 2) + " workgroups of 512 threads would not be resident together on this device");
  if (rc != 0) return fail(FX_E_HIP, std::string("fx_lstm_stack: ") + hipGetErrorString((hipError_t)(rc - 100)));
  g_launches.fetch_add(1, std::memory_order_relaxed);
  g_spec_launches.fetch_add(1, std::memory_order_relaxed);
  return FX_OK;
}
void fx_set_totals_spin_us(uint32_t us) { g_totals_spin_us.store(us, std::memory_order_relaxed); }
void fx_set_lstm_spin_limit(uint32_t polls) { g_lstm_spin.store(polls, std::memory_order_relaxed); }

// ---- detection tail (fx_nms.hip) ----

static uint32_t nms_key_cap(uint32_t want) {
  uint32_t cap = 128;
  while (cap < want) cap <<= 1;
  return cap;
}
size_t fx_sort_nms_workspace_bytes(int n_tasks, uint32_t key_capacity) {
  if (n_tasks < 1 || key_capacity < 1 || key_capacity > FX_NMS_MAX_CANDIDATES) return 0;
  return fx_nms_workspace_bytes(n_tasks, nms_key_cap(key_capacity));
}
size_t fx_sort_nms_workspace_clear_bytes(int n_tasks) { return n_tasks < 1 ? 0 : fx_nms_workspace_clear_bytes(n_tasks); }

int fx_sort_nms(const fx_nms_desc* desc, void* stream_) {
  if (!desc) return fail(FX_E_INVALID, "fx_sort_nms: null descriptor");
  fx_nms_desc d = *desc;
  if (d.mode != 0 && d.mode != 1) return fail(FX_E_INVALID, "fx_sort_nms: mode must be 0 or 1");
  if (d.n_tasks < 0) return fail(FX_E_INVALID, "fx_sort_nms: negative task count");
  if (!d.boxes || !d.scores || !d.dets || !d.out_labels || !d.n_out) return fail(FX_E_INVALID, "fx_sort_nms: null argument");
  if (((uintptr_t)d.boxes & 15u) != 0 || (d.boxes_task_stride & 3) != 0)
    return fail(FX_E_INVALID, "fx_sort_nms: boxes must be 16-byte aligned and their task stride a multiple of 4");
  if (d.max_num < 1 || d.max_num > FX_NMS_MAX_OUT)
    return fail(FX_E_LIMIT, "fx_sort_nms: max_num must be 1.." + std::to_string(FX_NMS_MAX_OUT));
  if (d.mode == 1 && d.n_classes < 1) return fail(FX_E_INVALID, "fx_sort_nms: n_classes must be positive in mode 1");
  if (d.mode == 0) d.scores_row_stride = 0;
  if (d.scores_row_stride != 0 && d.scores_row_stride < d.n_classes)
    return fail(FX_E_INVALID, "fx_sort_nms: scores_row_stride must be 0 or at least n_classes");
  const uint64_t items = (uint64_t)d.rows * (d.mode == 1 ? std::max(d.n_classes, d.scores_row_stride) : 1u);
  if (items >= (1ull << 31)) return fail(FX_E_LIMIT, "fx_sort_nms: rows * classes beyond 31 bits");
  if (d.key_capacity < 1 || d.key_capacity > FX_NMS_MAX_CANDIDATES)
    return fail(FX_E_LIMIT, "fx_sort_nms: key_capacity must be 1.." + std::to_string(FX_NMS_MAX_CANDIDATES) +
                                " (the reference's own single-pass branch ends at 10000 candidates)");
  if (d.n_tasks == 0) return FX_OK;
  const uint32_t cap = nms_key_cap(d.key_capacity);
  if (!d.workspace || ((uintptr_t)d.workspace & 255u) != 0 || d.workspace_bytes < fx_nms_workspace_bytes(d.n_tasks, cap))
    return fail(FX_E_INVALID, "fx_sort_nms: workspace must be 256-byte aligned and hold fx_sort_nms_workspace_bytes()");
  const int rc = fx_launch_sort_nms(d, cap, d.workspace, err_word(true), (hipStream_t)stream_);
  if (rc != 0) return fail(FX_E_HIP, std::string("fx_sort_nms: ") + hipGetErrorString((hipError_t)(rc - 100)));
  g_launches.fetch_add(1, std::memory_order_relaxed);
  g_spec_launches.fetch_add(1, std::memory_order_relaxed);
  return FX_OK;
}

int fx_copy_bytes(const void* src, void* dst, size_t bytes, void* stream) {
  if (bytes % 16) return fail(FX_E_INVALID, "fx_copy_bytes: size must be a multiple of 16");
  if (bytes == 0) return FX_OK;
  size_t n4 = bytes / 16;
  size_t blocks = (n4 + FX_BLOCK - 1) / FX_BLOCK;
  // 4 vectors per lane keeps enough loads in flight without oversubscribing; a small copy is
  // spread over as many workgroups as it has vectors for (4 MB: 2.9 us as 1024 workgroups, 4.4 us as 256)
  uint32_t grid = (uint32_t)std::min<size_t>(blocks <= 8192 ? blocks : (blocks + 3) / 4, 1u << 20);
  if (grid == 0) grid = 1;
  HIP_OK(fx_launch_copy(src, dst, bytes, grid, (hipStream_t)stream));
  return FX_OK;
}

int fx_copy_bytes_timed_sets(const void* const* src, void* const* dst, int n_sets, size_t bytes, int rounds, void* stream_,
                             float* ms_per_copy) {
  if (!src || !dst || !ms_per_copy || n_sets < 1 || rounds < 1) return fail(FX_E_INVALID, "fx_copy_bytes_timed_sets: bad argument");
  hipStream_t stream = (hipStream_t)stream_;
  for (int i = 0; i < n_sets; ++i) {   // (and every set once before the clock starts)
    const int rc = fx_copy_bytes(src[i], dst[i], bytes, stream_);
    if (rc != FX_OK) return rc;
  }
  hipEvent_t e0 = nullptr, e1 = nullptr;
  HIP_OK(hipEventCreate(&e0));
  HIP_OK(hipEventCreate(&e1));
  HIP_OK(hipEventRecord(e0, stream));
  int rc = FX_OK;
  for (int r = 0; r < rounds && rc == FX_OK; ++r)
    for (int i = 0; i < n_sets && rc == FX_OK; ++i) rc = fx_copy_bytes(src[i], dst[i], bytes, stream_);
  hipError_t e = hipEventRecord(e1, stream);
  if (e == hipSuccess) e = hipEventSynchronize(e1);
  float ms = 0.0f;
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (rc != FX_OK) return rc;
  HIP_OK(e);
  *ms_per_copy = ms / (float)((size_t)rounds * (size_t)n_sets);
  return FX_OK;
}

}  // extern "C"
