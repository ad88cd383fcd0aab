// Fused element-wise groups compiled at run time, one kernel per distinct program.
//
// The interpreting kernels of fused.hip decode each instruction for every vector of eight elements:
// scalar work that costs more than the arithmetic of a short chain.  Here the same program is
// written out as compile-time constants over the same device functions (fused_ops.cuh) and given
// to the run-time compiler once; the kernel is kept per context, keyed by what it is specialised on.  Same
// functions, same order, same flags (no contraction, no packed f32): bit-identical results.
// The device headers are embedded in the library as text, so nothing is read from disk.
#include <hip/hiprtc.h>

#include <algorithm>
#include <cstring>
#include <functional>
#include <string>
#include <vector>

#include "fused_ops.cuh"
#include "internal.h"
#include "rtc_headers.inc"

namespace hipnx {

// what the device headers take from host headers when the offline compiler builds them
static const char *const RTC_PREAMBLE = R"(
typedef unsigned char uint8_t; typedef signed char int8_t; typedef unsigned short uint16_t; typedef short int16_t;
typedef unsigned int uint32_t; typedef int int32_t; typedef unsigned long uint64_t; typedef long int64_t;
typedef unsigned long uintptr_t;
#define NAN __builtin_nanf("")
#define INFINITY __builtin_inff()
#define INT64_MAX 9223372036854775807L
#define INT64_MIN (-INT64_MAX - 1)
namespace std {
template <bool B, class T, class F> struct conditional { typedef T type; };
template <class T, class F> struct conditional<false, T, F> { typedef F type; };
template <class A, class B> struct is_same { static constexpr bool value = false; };
template <class A> struct is_same<A, A> { static constexpr bool value = true; };
template <class T> struct is_floating_point { static constexpr bool value = false; };
template <> struct is_floating_point<float> { static constexpr bool value = true; };
template <> struct is_floating_point<double> { static constexpr bool value = true; };
}
#include "fused_ops.cuh"
)";

static void list_of(std::string &s, const char *name, const char *type, int n, const std::function<std::string(int)> &at) {
  s += std::string("  static constexpr ") + type + " " + name + "[] = {";
  for (int i = 0; i < (n > 0 ? n : 1); i++) s += (i ? ", " : "") + (n > 0 ? at(i) : std::string("0"));
  s += "};\n";
}

// Trips of a lane along a row (of at most 4096 elements), when the program carries element values from
// stage to stage and so indexes their registers by the trip; 0 when it does not.
static int carry_trips(const FusedArgs &a) {
  for (int i = 0; i < a.n_instr; i++) {
    const hipnx_fused_instr &q = a.ins[i];
    const bool reads = q.kind == HIPNX_FUSED_SET || q.kind == HIPNX_FUSED_BINARY || q.kind == HIPNX_FUSED_SELECT;
    if (reads && (q.src == HIPNX_FUSED_SRC_CARRY || (q.kind == HIPNX_FUSED_SELECT && q.src2 == HIPNX_FUSED_SRC_CARRY)))
      {
        const int tpr = a.cols > 4096 ? FBLOCK : WAVE;
        const int64_t trips = (a.cols + tpr * FE - 1) / (tpr * FE);
        return trips <= 16 ? (int)trips : 0;  // (the host refuses longer rows for such programs)
      }
  }
  return 0;
}

// everything a compiled kernel is specialised on, as bytes: the cache key
static std::string make_key(const FusedArgs &a, int reduce_op, bool block_per_row) {
  std::string k;
  k.reserve(16 + 16 * a.n_instr + 8 * a.n_inputs);
  const int head[5] = {a.n_instr, a.n_inputs, a.out_dt, reduce_op * 2 + (block_per_row ? 1 : 0), carry_trips(a)};
  k.append((const char *)head, sizeof(head));
  k.append((const char *)a.ins, sizeof(hipnx_fused_instr) * a.n_instr);
  k.append((const char *)a.in_dt, sizeof(int) * a.n_inputs);
  k.append((const char *)a.in_cs, sizeof(int) * a.n_inputs);
  return k;
}

// the whole translation unit for one program
static std::string make_source(const FusedArgs &a, int reduce_op, bool block_per_row, const std::string &name) {
  std::string s = RTC_PREAMBLE;
  s += "namespace hipnx {\nstruct P {\n  static constexpr int n_instr = " + std::to_string(a.n_instr) + ", out_dt = " + std::to_string(a.out_dt) +
       ", nv = " + std::to_string(carry_trips(a)) + ", tpr = " + (block_per_row ? "FBLOCK" : "WAVE") + ";\n";
  const hipnx_fused_instr *q = a.ins;
  list_of(s, "kind", "int", a.n_instr, [&](int i) { return std::to_string((int)q[i].kind); });
  list_of(s, "op", "int", a.n_instr, [&](int i) { return std::to_string((int)q[i].op); });
  list_of(s, "src", "int", a.n_instr, [&](int i) { return std::to_string((int)q[i].src); });
  list_of(s, "arg", "int", a.n_instr, [&](int i) { return std::to_string((int)q[i].arg); });
  list_of(s, "src2", "int", a.n_instr, [&](int i) { return std::to_string((int)q[i].src2); });
  list_of(s, "arg2", "int", a.n_instr, [&](int i) { return std::to_string((int)q[i].arg2); });
  list_of(s, "flags", "int", a.n_instr, [&](int i) { return std::to_string((int)q[i].flags); });
  list_of(s, "dt", "int", a.n_instr, [&](int i) { return std::to_string((int)q[i].dt); });
  list_of(s, "imm", "unsigned", a.n_instr, [&](int i) { return std::to_string(q[i].imm_bits) + "u"; });
  list_of(s, "imm2", "unsigned", a.n_instr, [&](int i) { return std::to_string(q[i].imm2_bits) + "u"; });
  list_of(s, "in_dt", "int", a.n_inputs, [&](int k) { return std::to_string(a.in_dt[k]); });
  list_of(s, "in_cs", "int", a.n_inputs, [&](int k) { return std::to_string(a.in_cs[k]); });
  // stages: where each one's reduction and the end of its work on the statistic are (-1, n_instr for the last)
  std::vector<int> seg_red, seg_save;
  for (int i = 0; i < a.n_instr; i++) {
    if (q[i].kind == HIPNX_FUSED_ROW_REDUCE) seg_red.push_back(i);
    if (q[i].kind == HIPNX_FUSED_ROW_STAT) seg_save.push_back(i);
  }
  const bool stages = !seg_red.empty();
  if (seg_save.size() < seg_red.size() || seg_save.empty() || seg_save.back() != a.n_instr - 1) {  // a last, element-wise stage
    seg_red.push_back(-1);
    seg_save.push_back(a.n_instr);
  }
  list_of(s, "seg_red", "int", (int)seg_red.size(), [&](int k) { return std::to_string(seg_red[k]); });
  list_of(s, "seg_save", "int", (int)seg_save.size(), [&](int k) { return std::to_string(seg_save[k]); });
  s += "};\n}\nusing namespace hipnx;\nextern \"C\" __global__ void __launch_bounds__(FBLOCK) " + name + "(FusedArgs by_value) {\n  (void)by_value;\n";
  const char *tpr = block_per_row ? "FBLOCK" : "WAVE";
  if (stages) s += "  fused_row_stages_body<P>();\n";
  else switch (reduce_op) {
    case HIPNX_RED_SUM: s += std::string("  fused_reduce_rows_body<RunStatic<P>, PlainReducer<double, HIPNX_RED_SUM, false>, double, ") + tpr + ">();\n"; break;
    case HIPNX_RED_MAX: s += std::string("  fused_reduce_rows_body<RunStatic<P>, PlainReducer<float, HIPNX_RED_MAX, false>, float, ") + tpr + ">();\n"; break;
    case HIPNX_RED_MIN: s += std::string("  fused_reduce_rows_body<RunStatic<P>, PlainReducer<float, HIPNX_RED_MIN, false>, float, ") + tpr + ">();\n"; break;
    default: s += "  fused_elementwise_body<RunStatic<P>>();\n"; break;
  }
  s += "}\n";
  return s;
}

static int compile(hipnx_ctx *ctx, const std::string &src, const std::string &name, hipnx_ctx::FusedKernel *out) {
  hipDeviceProp_t prop;
  HIPNX_HIP(hipGetDeviceProperties(&prop, ctx->device));
  const std::string arch = std::string("--offload-arch=") + prop.gcnArchName;
  hiprtcProgram prog;
  if (hiprtcCreateProgram(&prog, src.c_str(), "fused_group.hip", RTC_NHEADERS, RTC_HEADER_SOURCES, RTC_HEADER_NAMES) != HIPRTC_SUCCESS)
    return set_error(HIPNX_EHIP, "fused: the run-time compiler did not take the program");
  const char *opts[] = {arch.c_str(), "-O3", "-std=c++17", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
  const hiprtcResult r = hiprtcCompileProgram(prog, (int)(sizeof(opts) / sizeof(opts[0])), opts);
  if (r != HIPRTC_SUCCESS) {
    size_t n = 0;
    hiprtcGetProgramLogSize(prog, &n);
    std::string log(n, '\0');
    if (n) hiprtcGetProgramLog(prog, &log[0]);
    hiprtcDestroyProgram(&prog);
    return set_error(HIPNX_EHIP, "fused: compiling a group failed (%s): %.600s", hiprtcGetErrorString(r), log.c_str());
  }
  size_t size = 0;
  hiprtcGetCodeSize(prog, &size);
  std::string code(size, '\0');
  hiprtcGetCode(prog, &code[0]);
  hiprtcDestroyProgram(&prog);
  HIPNX_HIP(hipModuleLoadData(&out->module, code.data()));
  hipError_t e = hipModuleGetFunction(&out->function, out->module, name.c_str());
  if (e != hipSuccess) {
    (void)hipModuleUnload(out->module);
    return hip_fail(e, "hipModuleGetFunction(fused group)");
  }
  return HIPNX_OK;
}

// Makes room in a full table: waits for the stream (a kernel may still be running), then unloads the least
// recently launched quarter.  A program specialised on a constant that changes from call to call (a
// temperature, a learning rate passed as a number) would otherwise grow the table, and the loaded
// modules with it, without bound; each new value still costs one compilation (a few hundred ms).
static int trim_cache(hipnx_ctx *ctx) {
  HIPNX_HIP(hipStreamSynchronize(ctx->stream));
  std::vector<std::pair<uint64_t, const std::string *>> by_age;
  for (auto &kv : ctx->fused_kernels)
    if (!kv.second.in_graph) by_age.emplace_back(kv.second.last_use, &kv.first);
  std::sort(by_age.begin(), by_age.end());
  // (a limit lowered below what is held: down to under the limit)
  const size_t over = ctx->fused_kernels.size() - ctx->fused_cache_max + 1;
  const size_t drop = std::min(by_age.size(), std::max<size_t>(over, ctx->fused_cache_max / 4));
  std::vector<std::string> keys;
  for (size_t i = 0; i < drop; i++) keys.push_back(*by_age[i].second);
  for (const std::string &k : keys) {
    auto it = ctx->fused_kernels.find(k);
    (void)hipModuleUnload(it->second.module);
    ctx->fused_kernels.erase(it);
  }
  return HIPNX_OK;
}

// Launches the compiled kernel for `a`, compiling it first if this context has not seen the program.
// *done = false (and HIPNX_OK) when the caller should run the interpreting kernel instead: the
// program is new and the stream is capturing (compiling and loading a module is no work to record).
int fused_launch_compiled(hipnx_ctx *ctx, const FusedArgs &a, int reduce_op, bool block_per_row, unsigned grid, bool *done) {
  *done = false;
  const std::string key = make_key(a, reduce_op, block_per_row);
  auto it = ctx->fused_kernels.find(key);
  if (it == ctx->fused_kernels.end()) {
    if (ctx->capture) return HIPNX_OK;
    // a name a profile can tell apart: what the kernel is (a map, a map with its row reduction, stages over rows),
    // how long its program is, and a hash of what it is specialised on
    int stages = 0;
    for (int i = 0; i < a.n_instr; i++) stages += a.ins[i].kind == HIPNX_FUSED_ROW_REDUCE;
    char name[96];
    snprintf(name, sizeof(name), "fused_%s_%dinstr_%08zx", stages ? "stages" : reduce_op != -1 ? "map_reduce" : "map", a.n_instr,
             std::hash<std::string>{}(key) & 0xFFFFFFFFu);
    if (ctx->fused_kernels.size() >= ctx->fused_cache_max)
      if (int st = trim_cache(ctx)) return st;
    hipnx_ctx::FusedKernel k{};
    if (int st = compile(ctx, make_source(a, reduce_op, block_per_row, name), name, &k)) return st;
    it = ctx->fused_kernels.emplace(key, k).first;
  }
  it->second.last_use = ++ctx->fused_clock;
  if (ctx->capture) it->second.in_graph = true;  // a recorded launch refers to the loaded module for as long as the graph lives
  // the argument block is the kernel's one by-value parameter: hand it over as the packed buffer it is
  size_t size = sizeof(FusedArgs);
  void *config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, (void *)&a, HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
  HIPNX_HIP(hipModuleLaunchKernel(it->second.function, grid, 1, 1, FBLOCK, 1, 1, 0, ctx->stream, nullptr, config));
  *done = true;
  return HIPNX_OK;
}

}  // namespace hipnx

using namespace hipnx;

extern "C" int hipnx_fused_set_mode(hipnx_ctx *ctx, int mode) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (mode != HIPNX_FUSED_INTERPRETED && mode != HIPNX_FUSED_COMPILED) return set_error(HIPNX_EINVAL, "fused: mode %d", mode);
  ctx->fused_mode = mode;
  return HIPNX_OK;
}

extern "C" int hipnx_fused_set_cache_limit(hipnx_ctx *ctx, int programs) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (programs < 4) return set_error(HIPNX_EINVAL, "fused: a cache limit of %d programs (at least 4)", programs);
  ctx->fused_cache_max = (size_t)programs;
  return HIPNX_OK;
}

extern "C" int hipnx_fused_compiled_count(hipnx_ctx *ctx, int *count) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (!count) return set_error(HIPNX_EINVAL, "fused: null count");
  *count = (int)ctx->fused_kernels.size();
  return HIPNX_OK;
}
