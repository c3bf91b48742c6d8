// Kernels specialised at run time: the MFMA GEMM template compiled by hipRTC for one configuration
// with the transform hooks given as C expressions.  This restores what the reference gets from its
// JIT: any elementwise functor at any of the eight hooks (src/transform.jl:20-30, src/matmul.jl:8-15)
// and block shapes outside the table compiled into the library (src/matmul.jl:38: one kernel per
// Config type).  The launch goes through the same host checks as gk_matmul.
#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>

#include "gk_internal.hpp"
#include "gk_embedded_headers.inc"

using gk_internal::fail;

struct gk_rtc_kernel {
  hipModule_t module = nullptr;
  hipFunction_t function = nullptr;
  gk::InstanceInfo info{};
  std::string name;
  int BM = 0, BN = 0, BK = 0, waves_m = 0, waves_n = 0, stages = 0, a_kmajor = 0, b_kmajor = 0, dtype = 0;
  int device = 0;
  bool lds_raised = false;
};

namespace {

// The run-time compiler ships the HIP device headers but no C++ standard library: the few standard
// templates the kernel headers use are declared here.
const char kPrelude[] =
    "typedef unsigned long long uintptr_t;\n"
    "namespace std {\n"
    "template <class T, T v> struct integral_constant { static constexpr T value = v; typedef T value_type; constexpr operator T() const { return v; } };\n"
    "typedef integral_constant<bool, true> true_type;\n"
    "typedef integral_constant<bool, false> false_type;\n"
    "template <class A, class B> struct is_same : false_type {};\n"
    "template <class A> struct is_same<A, A> : true_type {};\n"
    "}\n"
    // helpers for hook expressions, with the semantics of the library's op vocabulary
    "__device__ __forceinline__ float gk_relu(float x) { return x > 0.0f ? x : 0.0f; }\n"
    "__device__ __forceinline__ float gk_abs(float x) { return __builtin_fabsf(x); }\n"
    "__device__ __forceinline__ float gk_clamp(float x, float lo, float hi) { return x < lo ? lo : (x > hi ? hi : x); }\n"
    "__device__ __forceinline__ float gk_square(float x) { return x * x; }\n";

const char* const kHookNames[8] = {"global_to_shared_a", "global_to_shared_b", "global_to_shared_c", "shared_to_global_d",
                                   "shared_to_regs_a",   "shared_to_regs_b",   "shared_to_regs_c",   "regs_to_shared_d"};

bool is_row_major(int kind) { return kind == GK_LAYOUT_ROW_MAJOR || kind == GK_LAYOUT_ALIGNED_ROW_MAJOR; }

// LDS stages of a run-time tile: as many as fit the 160 KiB of a CU, between 2 and 4, and few enough
// for the 6-bit counter of outstanding loads the pipeline waits on.
int pick_stages(int BM, int BN, int BK, int nwaves) {
  const long long stage = (long long)(BM + BN) * BK * 2;
  const int dma_per_tile = (int)(stage / 1024 / nwaves);
  int s = (int)((160 * 1024) / stage);
  if (s > 4) s = 4;
  while (s > 2 && (s - 2) * dma_per_tile > 63) --s;
  return s;
}

std::mutex g_mutex;
std::unordered_map<std::string, gk_rtc_kernel*> g_cache;      // source text + device -> kernel

std::string build_source(const gk_config* c, const char* const hooks[8], int stages, int fuse, int a_kind, int b_kind, const char* type) {
  std::string src = "#define GK_USER_HOOKS 1\n";
  src += kPrelude;
  src += "namespace gk {\nstruct UserHooks {\n  static constexpr bool present[8] = {";
  for (int h = 0; h < 8; ++h) src += (hooks && hooks[h] && hooks[h][0]) ? (h ? ", true" : "true") : (h ? ", false" : "false");
  src += "};\n  template <int H> static __device__ __forceinline__ float apply(float x) {\n";
  for (int h = 0; h < 8; ++h)
    if (hooks && hooks[h] && hooks[h][0]) {
      src += "    if constexpr (H == " + std::to_string(h) + ") { return (" + hooks[h] + "); }   // " + kHookNames[h] + "\n";
    }
  src += "    return x;\n  }\n};\n}\n#include \"mfma_gemm.hpp\"\n";
  char buf[512];
  snprintf(buf, sizeof(buf),
           "typedef gk::MfmaGemmConfig<%d, %d, %d, %d, %d, %d, %d, %d, %s, %d, false, gk::FIX_NONE, false, %d> GkUserCfg;\n"
           "template __global__ void gk::mfma_gemm_kernel<GkUserCfg>(const gk::GemmArgs);\n",
           c->block_shape.M, c->block_shape.N, c->block_shape.K, c->block_shape.M / c->compute_warp.M,
           c->block_shape.N / c->compute_warp.N, stages, a_kind, b_kind, type, fuse,
           // v_mfma_f32_16x16x32 takes 32 values of k at a time; a BLOCK_K of 16 (the reference sweeps it,
           // configs/configs.jl:601) runs on v_mfma_f32_32x32x16
           c->block_shape.K % 32 == 0 ? 16 : 32);
  src += buf;
  return src;
}

}  // namespace

extern "C" {

int gk_rtc_compile(const gk_config* conf, const char* const hooks[8], int32_t kernel, gk_rtc_kernel** out) {
  if (!conf || !out) return fail(GK_ERR_INVALID_ARGUMENT, "conf and out must not be NULL");
  *out = nullptr;
  (void)kernel;
  const gk_config* c = conf;
  if (c->op.kind != GK_OP_MFMA) return fail(GK_ERR_UNSUPPORTED, "run-time specialisation is offered for the real MFMA operator");
  const gk_layout* ls[4] = {&c->global_a_layout, &c->global_b_layout, &c->global_c_layout, &c->global_d_layout};
  for (const gk_layout* l : ls)
    if (l->kind != GK_LAYOUT_ALIGNED_COL_MAJOR && l->kind != GK_LAYOUT_ALIGNED_ROW_MAJOR && l->kind != GK_LAYOUT_ZERO)
      return fail(GK_ERR_UNSUPPORTED, "run-time specialisation needs aligned (or Zero) global layouts");
  const int dt = c->global_a_layout.eltype;
  if ((dt != GK_F16 && dt != GK_BF16) || c->global_b_layout.eltype != dt)
    return fail(GK_ERR_UNSUPPORTED, "run-time specialisation takes Float16 or BFloat16 multiplicands");
  const gk_shape& b = c->block_shape;
  const gk_shape& w = c->compute_warp;
  if (b.M <= 0 || b.N <= 0 || b.K <= 0 || w.M <= 0 || w.N <= 0 || b.M % w.M || b.N % w.N)
    return fail(GK_ERR_BLOCK_SHAPE, "block_shape must be a positive multiple of compute_warp");
  const int wm = b.M / w.M, wn = b.N / w.N, nwaves = wm * wn;
  if (w.M % 32 || w.N % 32 || (b.K != 16 && b.K % 32) || b.K > 128) return fail(GK_ERR_BLOCK_SHAPE, "compute_warp must be made of 32x32 blocks and BLOCK_K be 16, 32, 64 or 128");
  if ((w.M / 32) * (w.N / 32) > 16) return fail(GK_ERR_BLOCK_SHAPE, "a wave tile holds at most sixteen 32x32 accumulator blocks");
  if (nwaves > 16 || nwaves != c->warps_per_block) return fail(GK_ERR_UNSUPPORTED, "warps_per_block must equal block_shape / compute_warp (at most 16)");
  if (((long long)b.M * b.K * 2 / 1024) % nwaves || ((long long)b.N * b.K * 2 / 1024) % nwaves || ((long long)b.M * b.K * 2) % 1024 || ((long long)b.N * b.K * 2) % 1024)
    return fail(GK_ERR_BLOCK_SHAPE, "every wave must move the same whole number of 1 KiB pieces of the A tile and of the B tile");
  const int stages = pick_stages(b.M, b.N, b.K, nwaves);
  if (stages < 2) return fail(GK_ERR_LDS, "two stages of this block shape do not fit the 160 KiB of LDS");
  const int a_kmajor = is_row_major(c->global_a_layout.kind) ? 1 : 0;     // 'T' A: stored K x M, K contiguous
  const int b_kmajor = is_row_major(c->global_b_layout.kind) ? 0 : 1;     // 'N' B: stored K x N, K contiguous
  if ((!a_kmajor && (b.M & (b.M - 1))) || (!b_kmajor && (b.N & (b.N - 1))))
    return fail(GK_ERR_BLOCK_SHAPE, "an operand that is contiguous along M (N) needs a power-of-two BLOCK_M (BLOCK_N)");
  bool any_ab = false, any = false;
  for (int h = 0; h < 8; ++h)
    if (hooks && hooks[h] && hooks[h][0]) {
      any = true;
      if (h == GK_HOOK_GLOBAL_TO_SHARED_A || h == GK_HOOK_GLOBAL_TO_SHARED_B || h == GK_HOOK_SHARED_TO_REGS_A || h == GK_HOOK_SHARED_TO_REGS_B) any_ab = true;
      if (strlen(hooks[h]) > 1024) return fail(GK_ERR_INVALID_ARGUMENT, "hook expression longer than 1024 characters");
    }
  (void)any;
  const int fuse = any_ab ? 2 : 1;      // level 1 also carries the bias epilogue, chosen at launch time
  // operand kinds of the kernel template: 0 K-major, 1 M-major
  const std::string src = build_source(c, hooks, stages, fuse, a_kmajor ? 0 : 1, b_kmajor ? 0 : 1, dt == GK_F16 ? "_Float16" : "__bf16");

  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) { (void)hipGetLastError(); device = -1; }     // compile-only use without a GPU
  const std::string cache_key = std::to_string(device) + "\n" + src;
  std::lock_guard<std::mutex> lock(g_mutex);
  auto hit = g_cache.find(cache_key);
  if (hit != g_cache.end()) { *out = hit->second; return GK_OK; }

  // compiles one source text; the code object and the mangled kernel name come back
  auto compile = [](const std::string& text, std::string& code, std::string& lowered_name) -> int {
    hiprtcProgram prog;
    const char* header_names[2] = {"common.hpp", "mfma_gemm.hpp"};
    const char* header_text[2] = {kEmbedded_common_hpp, kEmbedded_mfma_gemm_hpp};
    hiprtcResult r = hiprtcCreateProgram(&prog, text.c_str(), "gk_user_kernel.hip", 2, header_text, header_names);
    if (r != HIPRTC_SUCCESS) return fail(GK_ERR_HIP, "hiprtcCreateProgram: %s", hiprtcGetErrorString(r));
    const char* name_expr = "&gk::mfma_gemm_kernel<GkUserCfg>";
    hiprtcAddNameExpression(prog, name_expr);
    const char* opts[] = {"--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off"};
    r = hiprtcCompileProgram(prog, 4, opts);
    if (r != HIPRTC_SUCCESS) {
      size_t n = 0;
      hiprtcGetProgramLogSize(prog, &n);
      std::string log(n ? n : 1, '\0');
      if (n) hiprtcGetProgramLog(prog, &log[0]);
      hiprtcDestroyProgram(&prog);
      // a failed static_assert of the tile geometry or a malformed expression: the compiler says which
      return fail(GK_ERR_UNSUPPORTED, "run-time compilation failed: %.1800s", log.c_str());
    }
    const char* lowered = nullptr;
    r = hiprtcGetLoweredName(prog, name_expr, &lowered);
    size_t code_size = 0;
    if (r == HIPRTC_SUCCESS) r = hiprtcGetCodeSize(prog, &code_size);
    code.assign(code_size, '\0');
    if (r == HIPRTC_SUCCESS) r = hiprtcGetCode(prog, &code[0]);
    lowered_name = lowered ? lowered : "";
    hiprtcDestroyProgram(&prog);
    if (r != HIPRTC_SUCCESS || lowered_name.empty()) return fail(GK_ERR_HIP, "hipRTC produced no code object: %s", hiprtcGetErrorString(r));
    return GK_OK;
  };
  std::string code, lowered_name;
  int rc_compile = compile(src, code, lowered_name);
  if (rc_compile != GK_OK) return rc_compile;

  gk_rtc_kernel* k = new gk_rtc_kernel();
  k->BM = b.M; k->BN = b.N; k->BK = b.K; k->waves_m = wm; k->waves_n = wn; k->stages = stages;
  k->a_kmajor = a_kmajor; k->b_kmajor = b_kmajor; k->dtype = dt; k->device = device;
  char nm[160];
  snprintf(nm, sizeof(nm), "mfma_gemm_rtc_%c%c_%dx%dx%d_w%dx%d_s%d_%s", a_kmajor ? 't' : 'n', b_kmajor ? 'n' : 't', b.M, b.N, b.K, wm, wn,
           stages, dt == GK_F16 ? "f16" : "bf16");
  k->name = nm;
  k->info.name = k->name.c_str();
  k->info.lds_bytes = (int)((long long)(b.M + b.N) * b.K * 2 * stages);
  k->info.threads = nwaves * gk::kWaveSize;
  if (device >= 0) {
    auto load = [&]() -> hipError_t {
      hipError_t e = hipModuleLoadData(&k->module, code.data());
      if (e == hipSuccess) e = hipModuleGetFunction(&k->function, k->module, lowered_name.c_str());
      return e;
    };
    hipError_t e = load();
    // The fragment reads of the kernel are asynchronous with hand-placed waits, which is sound only
    // while no register is spilled (a spill store between a read and its wait would save stale
    // values).  A tile that makes this kernel use scratch memory is compiled again with reads that
    // wait inside the assembly statement that issues them.
    const bool sync_already = fuse == 2 || (w.M / 32) * (w.N / 32) > 8;     // MfmaGemmConfig::SYNC_FRAGS
    int scratch_bytes = 0;
    if (e == hipSuccess && !sync_already &&
        hipFuncGetAttribute(&scratch_bytes, HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES, k->function) == hipSuccess && scratch_bytes > 0) {
      (void)hipModuleUnload(k->module);
      k->module = nullptr;
      k->function = nullptr;
      int rc2 = compile("#define GK_FORCE_SYNC_FRAGS 1\n" + src, code, lowered_name);
      if (rc2 != GK_OK) { delete k; return rc2; }
      e = load();
      k->name += "_sync";
      k->info.name = k->name.c_str();
    }
    if (e != hipSuccess) {
      if (k->module) (void)hipModuleUnload(k->module);
      delete k;
      return fail(GK_ERR_HIP, "loading the compiled kernel failed: %s", hipGetErrorString(e));
    }
  }
  g_cache.emplace(cache_key, k);
  *out = k;
  return GK_OK;
}

int gk_rtc_kernel_name(const gk_rtc_kernel* k, char* buf, size_t n) {
  if (!k || !buf || n == 0) return fail(GK_ERR_INVALID_ARGUMENT, "NULL argument");
  snprintf(buf, n, "%s", k->name.c_str());
  return GK_OK;
}

int gk_rtc_matmul(gk_rtc_kernel* k, const gk_config* conf, const void* a, const void* b, const void* c, void* d,
                  const gk_epilogue* epilogue, void* stream) {
  if (!k || !conf) return fail(GK_ERR_INVALID_ARGUMENT, "kernel and conf must not be NULL");
  if (!k->function) return fail(GK_ERR_HIP, "this kernel was compiled without a GPU and cannot be launched");
  const gk_shape& bs = conf->block_shape;
  const int a_kmajor = is_row_major(conf->global_a_layout.kind) ? 1 : 0, b_kmajor = is_row_major(conf->global_b_layout.kind) ? 0 : 1;
  if (bs.M != k->BM || bs.N != k->BN || bs.K != k->BK || conf->compute_warp.M * k->waves_m != bs.M || conf->compute_warp.N * k->waves_n != bs.N ||
      a_kmajor != k->a_kmajor || b_kmajor != k->b_kmajor || conf->global_a_layout.eltype != k->dtype || conf->op.kind != GK_OP_MFMA)
    return fail(GK_ERR_INVALID_ARGUMENT, "the configuration differs from the one this kernel was compiled for");
  {
    // the same rule as at compile time: whole tiles on aligned layouts (the bounds-checked layouts would let
    // sizes through that this kernel cannot mask)
    const gk_layout* ls[4] = {&conf->global_a_layout, &conf->global_b_layout, &conf->global_c_layout, &conf->global_d_layout};
    for (const gk_layout* l : ls)
      if (l->kind != GK_LAYOUT_ALIGNED_COL_MAJOR && l->kind != GK_LAYOUT_ALIGNED_ROW_MAJOR && l->kind != GK_LAYOUT_ZERO)
        return fail(GK_ERR_UNSUPPORTED, "run-time specialisation needs aligned (or Zero) global layouts");
  }
  // a bias epilogue makes the host layer choose a fused path; the hooks themselves are compiled in,
  // so no op lists travel with the launch
  gk_internal::Launch L;
  // (a block that is a single operator k-step deep -- BLOCK_K = 16 -- is what the reference can only run on its
  // single-stage kernel, src/matmul.jl:34-36; the compiled code is the same pipeline either way)
  const int kind = conf->block_shape.K < 2 * conf->compute_op_shape.K ? GK_KERNEL_SINGLESTAGE : GK_KERNEL_PIPELINED;
  int rc = gk_internal::prepare_launch(conf, a, b, c, d, nullptr, epilogue, kind, &k->info, &L);
  if (rc != GK_OK) return rc;
  L.args.fast_scale_a = L.args.fast_scale_b = 0;
  if (k->info.lds_bytes > 64 * 1024 && !k->lds_raised) {
    // module functions take the attribute through the same call as host-side kernel symbols; a
    // runtime that does not accept it for them reports the LDS request at the launch below instead
    if (hipFuncSetAttribute((const void*)k->function, hipFuncAttributeMaxDynamicSharedMemorySize, k->info.lds_bytes) != hipSuccess)
      (void)hipGetLastError();
    k->lds_raised = true;
  }
  size_t arg_size = sizeof(L.args);
  void* launch_config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, &L.args, HIP_LAUNCH_PARAM_BUFFER_SIZE, &arg_size, HIP_LAUNCH_PARAM_END};
  hipError_t e = hipModuleLaunchKernel(k->function, (unsigned)L.gx, (unsigned)L.gy, 1, (unsigned)k->info.threads, 1, 1,
                                       (unsigned)k->info.lds_bytes, (hipStream_t)stream, nullptr, launch_config);
  if (e != hipSuccess) return fail(GK_ERR_HIP, "launch of %s failed: %s", k->name.c_str(), hipGetErrorString(e));
  return GK_OK;
}

}  // extern "C"
