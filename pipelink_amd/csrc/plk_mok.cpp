// Implementation of include/plk_mok.h: host side of the routed-expert MXFP8 FFN forward.
// Builds the params image the linked pipeline kernel reads (framework schedule params,
// GEMM residue, activation residue at their linked offsets), keeps it resident on the
// device, and launches the gate/up pass and the down pass.
#include "plk_mok.h"

#include <hip/hip_runtime.h>

#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "plk_mok_residues.hpp"

extern "C" int plk_hip_set_error(int code, const char* what);

using plk_mok::NUM_XCD;

constexpr int IMAGES = 3;  // params images a session keeps: both GEMMs in one launch (pass 0), pass 1, pass 2

struct plk_mok_session {
  plk_hip_module* module = nullptr;
  plk_hip_function* kernel = nullptr;
  plk_mok_link_info link{};
  uint64_t params_dev[IMAGES] = {0, 0, 0};         // device copies of the params images, by pass
  std::vector<unsigned char> params_host[IMAGES];  // what the device copies hold
  uint64_t workspace = 0;                          // readiness counters of a launch (device, zero between launches)
  int64_t workspace_words = 0;
  int32_t compute_units = 0;
  int device = 0;  // the device that was current when the session was created
  bool used_static = false;  // plk_mok_forward_static has run: the static area's status word counts too
  uint32_t carried_status = 0;  // status bits of a workspace that has been replaced since: plk_mok_status reports them
  bool two_launches = false;    // plk_mok_forward runs pass 1 then pass 2 (asked for, or a one-launch forward gave up a wait)
};

// words the session's first workspace is made for (a problem that needs more gets a larger one)
constexpr int64_t WORKSPACE_WORDS_AT_CREATE = 4096;

static plk_mok::Dims dims_of(const plk_mok_problem* p, int pass) {
  plk_mok::Dims d;
  d.tokens = p->num_tokens;
  d.hidden = p->hidden;
  d.intermediate = p->intermediate;
  d.experts = p->num_experts;
  d.routed_rows = p->routed_rows;
  d.ld_q_h = p->ld_q_h ? p->ld_q_h : p->hidden;
  d.ld_q_i = p->ld_q_i ? p->ld_q_i : p->intermediate;
  d.ld_sc_h = p->ld_sc_h;
  d.ld_sc_i = p->ld_sc_i;
  d.pass = pass;
  d.swiglu_limit = p->swiglu_limit;
  return d;
}

static int check_problem(const plk_mok_problem* p) {
  if (!p || p->struct_bytes != sizeof(plk_mok_problem))
    return plk_hip_set_error(PLK_E_VERSION, "plk_mok: problem struct size mismatch");
  const plk_mok::Dims d = dims_of(p, 1);
  if (const char* what = plk_mok::check_dims(d)) {
    static thread_local std::string msg;
    msg = std::string("plk_mok: ") + what;
    const bool capacity = d.experts <= 0 || d.experts > plk_mok::MAX_EXPERTS || msg.find("4 GiB") != std::string::npos;
    return plk_hip_set_error(capacity ? PLK_E_CAPACITY : PLK_E_ARGUMENT, msg.c_str());
  }
  if (p->routed_rows && (!p->x_q || !p->x_sc || !p->tokens_per_expert || !p->w_gate_q || !p->w_gate_sc ||
                         !p->w_up_q || !p->w_up_sc || !p->w_down_q || !p->w_down_sc || !p->hidden_q ||
                         !p->hidden_sc || !p->y))
    return plk_hip_set_error(PLK_E_ARGUMENT, "plk_mok: null device address");
  return PLK_OK;
}


static bool stream_is_capturing(void* stream) {
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  return stream && hipStreamIsCapturing((hipStream_t)stream, &capturing) == hipSuccess && capturing == hipStreamCaptureStatusActive;
}

// (re)places the session's workspace by one of at least `words` zeroed words.  Everything the device is doing ends
// first (launches on any stream may use the old one), and the status bits the old one holds stay with the session.
static int make_workspace(plk_mok_session* s, int64_t words) {
  if (s->workspace) {
    if (hipDeviceSynchronize() != hipSuccess) return plk_hip_set_error(PLK_E_RESOURCE, "plk_mok: device synchronisation failed");
    uint32_t word = 0;
    int rc = plk_hip_readback(&word, s->workspace + MOK_WS_STATUS * 4, sizeof word, nullptr);
    if (rc == PLK_OK) s->carried_status |= word;
    const int rc_free = plk_hip_free(s->workspace);  // (freed whether or not its status could be read)
    if (rc == PLK_OK) rc = rc_free;
    s->workspace = 0;
    s->workspace_words = 0;
    if (rc != PLK_OK) return rc;
  }
  int rc = plk_hip_alloc((size_t)words * 4, &s->workspace);
  if (rc == PLK_OK) rc = plk_hip_zero(s->workspace, (size_t)words * 4, nullptr);
  if (rc == PLK_OK) rc = plk_hip_synchronize(nullptr);
  if (rc == PLK_OK) s->workspace_words = words;
  return rc;
}

// One pass's params image: the three owners' records at their linked offsets, zeros between them.
static void fill_image(const plk_mok_link_info& link, const plk_mok_problem* p, int pass, uint64_t workspace, unsigned char* image) {
  const plk_mok::Dims d = dims_of(p, pass);
  const MokFrameworkParams fw = plk_mok::framework_params(d, p->tokens_per_expert, workspace);
  const MokGemmResidue g = plk_mok::gemm_residue(
      d, plk_mok::GemmAddresses{p->x_q, p->x_sc, p->w_gate_q, p->w_gate_sc, p->w_up_q, p->w_up_sc, p->w_down_q, p->w_down_sc,
                                p->hidden_q, p->hidden_sc, p->y, p->row_token});
  const MokActResidue a = plk_mok::act_residue(d, p->hidden_q, p->hidden_sc);
  std::memcpy(image + link.framework_offset, &fw, sizeof fw);
  std::memcpy(image + link.gemm_offset, &g, sizeof g);
  std::memcpy(image + link.act_offset, &a, sizeof a);
}

// Launch of one pass on a params image that is already on the device.  Persistent grid: the solved occupancy
// on every CU, a multiple of the XCD count, but no more workgroups than there can be tiles.
static int launch_pass(plk_mok_session* s, const plk_mok_problem* p, int pass, void* stream, uint64_t params_dev) {
  const plk_mok::Dims d = dims_of(p, pass);
  const int64_t max_tiles = plk_mok::max_workgroups(d);
  int64_t wgs = (int64_t)s->compute_units * s->link.workgroups_per_cu;
  if (wgs > max_tiles) wgs = max_tiles;
  wgs = (wgs + NUM_XCD - 1) / NUM_XCD * NUM_XCD;
  const uint32_t grid[3] = {(uint32_t)wgs, 1, 1};
  const uint32_t block[3] = {s->link.threads, 1, 1};
  return plk_hip_launch(s->kernel, grid, block, s->link.dyn_lds_bytes, stream, params_dev);
}

// ---- device memory of the entry point that allocates nothing (plk_mok_forward_static) -------------------
// What plk_mok_forward keeps in buffers the session allocates -- the params images of the launches (two at most,
// PLK_MOK_STATIC_IMAGE_BYTES each) and the launch workspace (status word and readiness counters, up to
// PLK_MOK_STATIC_WORKSPACE_WORDS words) -- lives in this file-scope array: every GPU the library runs on holds its
// own copy, at its own address, until the process ends.  `scratch` is only a name on the host; the address
// kernels are given is what hipGetSymbolAddress returned for the device that was current, kept per device in
// g_static_area.
constexpr int STATIC_IMAGE_WORDS = 2 * PLK_MOK_STATIC_IMAGE_BYTES / 4;
constexpr size_t STATIC_WORKSPACE_OFFSET = 2 * PLK_MOK_STATIC_IMAGE_BYTES;
static __device__ __align__(256) unsigned char scratch[STATIC_WORKSPACE_OFFSET + 4 * PLK_MOK_STATIC_WORKSPACE_WORDS];
constexpr int MAX_DEVICES = 64;
static unsigned char* g_static_area[MAX_DEVICES];
static std::mutex g_static_mutex;

struct StaticImages {
  uint32_t words[STATIC_IMAGE_WORDS];
};
// Stores the params images and puts the workspace words a launch of this size uses back to zero (a launch leaves them
// zero, but one that was cut short would not have); word 0, the sticky status, is left alone.
__global__ void __launch_bounds__(STATIC_IMAGE_WORDS) plk_mok_store_images(StaticImages images, uint32_t* dst, uint32_t* workspace,
                                                                           int workspace_words) {
  dst[threadIdx.x] = images.words[threadIdx.x];
  for (int w = 1 + threadIdx.x; w < workspace_words; w += STATIC_IMAGE_WORDS) workspace[w] = 0u;
}

// once per device, with that device current
static int resolve_static_area(int dev) {
  if (dev < 0 || dev >= MAX_DEVICES) return plk_hip_set_error(PLK_E_CAPACITY, "plk_mok: device ordinal beyond 63");
  std::lock_guard<std::mutex> lock(g_static_mutex);
  if (g_static_area[dev]) return PLK_OK;
  void* ptr = nullptr;
  const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !ptr) {
    (void)hipGetLastError();
    return plk_hip_set_error(PLK_E_RESOURCE, "plk_mok: hipGetSymbolAddress of the static params area failed");
  }
  g_static_area[dev] = static_cast<unsigned char*>(ptr);
  return PLK_OK;
}

extern "C" {

int plk_mok_session_create(const void* image, size_t image_bytes, const plk_mok_link_info* link,
                           plk_mok_session** out) {
  if (!image || !link || !out) return plk_hip_set_error(PLK_E_ARGUMENT, "plk_mok_session_create: null argument");
  if (link->struct_bytes != sizeof(plk_mok_link_info))
    return plk_hip_set_error(PLK_E_VERSION, "plk_mok_session_create: link info struct size mismatch");
  const uint32_t need[3][2] = {{link->framework_offset, (uint32_t)sizeof(MokFrameworkParams)},
                               {link->gemm_offset, (uint32_t)sizeof(MokGemmResidue)},
                               {link->act_offset, (uint32_t)sizeof(MokActResidue)}};
  for (auto& n : need)
    if (n[0] % 8 || n[0] + n[1] > link->params_bytes)
      return plk_hip_set_error(PLK_E_CONTRACT, "plk_mok_session_create: params entry outside the image or misaligned");
  if (link->threads != 256) return plk_hip_set_error(PLK_E_CONTRACT, "plk_mok_session_create: image must use 256 threads");
  auto* s = new plk_mok_session;
  s->link = *link;
  int rc = plk_hip_module_load(image, image_bytes, &s->module);
  if (rc == PLK_OK) rc = plk_hip_module_function(s->module, "pipelink_kernel", link->dyn_lds_bytes, &s->kernel);
  for (int i = 0; i < IMAGES && rc == PLK_OK; ++i) {
    rc = plk_hip_alloc(link->params_bytes, &s->params_dev[i]);
    s->params_host[i].assign(link->params_bytes, 0xA5);  // differs from any real image: first call uploads
  }
  if (rc == PLK_OK) rc = make_workspace(s, WORKSPACE_WORDS_AT_CREATE);
  if (rc == PLK_OK) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 0;
    plk_hip_device_info info;
    rc = plk_hip_device_info_get(dev, &info);
    s->compute_units = info.compute_units;
    s->device = dev;
    if (rc == PLK_OK) rc = resolve_static_area(dev);
  }
  if (rc != PLK_OK) {
    plk_mok_session_destroy(s);
    return rc;
  }
  *out = s;
  return PLK_OK;
}

int plk_mok_session_destroy(plk_mok_session* s) {
  if (!s) return PLK_OK;
  int rc = PLK_OK;
  for (uint64_t a : s->params_dev)
    if (a) { int r = plk_hip_free(a); if (r) rc = r; }
  if (s->workspace) { int r = plk_hip_free(s->workspace); if (r) rc = r; }
  if (s->module) { int r = plk_hip_module_unload(s->module); if (r) rc = r; }
  delete s;
  return rc;
}

// One launch of the session's image: pass 0 = both GEMMs, 1 = gate/up + SwiGLU + requant, 2 = down.
static int forward_launch(plk_mok_session* s, const plk_mok_problem* p, int pass, void* stream) {
  const plk_mok::Dims d = dims_of(p, pass);
  int rc = PLK_OK;
  if (plk_mok::workspace_words(d) > s->workspace_words) {
    // a larger problem than any before: the launches that use the present workspace end first
    if (stream_is_capturing(stream))
      return plk_hip_set_error(PLK_E_CONTRACT, "plk_mok_forward: this problem needs a larger workspace; run the forward once "
                                               "before capturing it into a graph");
    rc = make_workspace(s, plk_mok::workspace_words(d));
    if (rc != PLK_OK) return rc;
  }
  std::vector<unsigned char> image(s->link.params_bytes, 0);
  fill_image(s->link, p, pass, s->workspace, image.data());
  if (image != s->params_host[pass]) {
    // a new problem: its params image goes to the device first, which synchronises and cannot be part of a graph
    if (stream_is_capturing(stream))
      return plk_hip_set_error(PLK_E_CONTRACT, "plk_mok_forward: this problem's params image is not on the device yet; run the "
                                               "forward once before capturing it into a graph");
    rc = plk_hip_upload(s->params_dev[pass], image.data(), image.size(), stream);
    if (rc != PLK_OK) return rc;
    s->params_host[pass].swap(image);
  }
  return launch_pass(s, p, pass, stream, s->params_dev[pass]);
}

int plk_mok_forward_pass(plk_mok_session* s, const plk_mok_problem* p, int pass, void* stream) {
  if (!s) return plk_hip_set_error(PLK_E_ARGUMENT, "plk_mok_forward: null session");
  if (pass != 1 && pass != 2) return plk_hip_set_error(PLK_E_ARGUMENT, "plk_mok_forward: pass must be 1 or 2");
  int rc = check_problem(p);
  if (rc != PLK_OK) return rc;
  if (p->routed_rows == 0) return PLK_OK;  // nothing routed to this rank
  return forward_launch(s, p, pass, stream);
}

int plk_mok_forward(plk_mok_session* s, const plk_mok_problem* p, void* stream) {
  if (!s) return plk_hip_set_error(PLK_E_ARGUMENT, "plk_mok_forward: null session");
  int rc = check_problem(p);
  if (rc != PLK_OK) return rc;
  if (p->routed_rows == 0) return PLK_OK;
  if (!s->two_launches && plk_mok::one_launch_ok(dims_of(p, 0), p->hidden_q)) return forward_launch(s, p, 0, stream);
  rc = forward_launch(s, p, 1, stream);  // the launch boundary orders the two GEMMs
  if (rc == PLK_OK) rc = forward_launch(s, p, 2, stream);
  return rc;
}

int plk_mok_status(plk_mok_session* s, void* stream, uint32_t* status) {
  if (!s || !status) return plk_hip_set_error(PLK_E_ARGUMENT, "plk_mok_status: null argument");
  uint32_t word = 0;
  int rc = plk_hip_readback(&word, s->workspace + MOK_WS_STATUS * 4, sizeof word, stream);  // waits for the stream
  if (rc != PLK_OK) return rc;
  if (word) rc = plk_hip_zero(s->workspace + MOK_WS_STATUS * 4, sizeof word, stream);
  if (rc == PLK_OK && s->used_static && g_static_area[s->device]) {
    const uint64_t at = (uint64_t)(uintptr_t)(g_static_area[s->device] + STATIC_WORKSPACE_OFFSET) + MOK_WS_STATUS * 4;
    uint32_t other = 0;
    rc = plk_hip_readback(&other, at, sizeof other, stream);
    if (rc == PLK_OK && other) rc = plk_hip_zero(at, sizeof other, stream);
    word |= other;
  }
  word |= s->carried_status;
  s->carried_status = 0;
  // A wait gave up: the GPU is not this session's alone (or the launch was larger than what can be resident).  From
  // here on the forward is two launches, which depend on nothing inside a launch.
  if (word & MOK_STATUS_WAIT_GAVE_UP) s->two_launches = true;
  *status = word;
  return rc;
}

int plk_mok_session_launches(plk_mok_session* s, int launches) {
  if (!s) return plk_hip_set_error(PLK_E_ARGUMENT, "plk_mok_session_launches: null session");
  if (launches != 1 && launches != 2) return plk_hip_set_error(PLK_E_ARGUMENT, "plk_mok_session_launches: 1 or 2");
  s->two_launches = launches == 2;
  return PLK_OK;
}

int plk_mok_forward_static(plk_mok_session* s, const plk_mok_problem* p, void* stream) {
  if (!s) return plk_hip_set_error(PLK_E_ARGUMENT, "plk_mok_forward_static: null session");
  int rc = check_problem(p);
  if (rc != PLK_OK) return rc;
  if (s->link.params_bytes > PLK_MOK_STATIC_IMAGE_BYTES)
    return plk_hip_set_error(PLK_E_CAPACITY, "plk_mok_forward_static: the linked image's params exceed "
                                             "PLK_MOK_STATIC_IMAGE_BYTES (1024) per launch");
  const int64_t words = plk_mok::workspace_words(dims_of(p, 0));
  if (words > PLK_MOK_STATIC_WORKSPACE_WORDS)
    return plk_hip_set_error(PLK_E_CAPACITY, "plk_mok_forward_static: routed_rows / 256 + num_experts + 32 exceeds "
                                             "PLK_MOK_STATIC_WORKSPACE_WORDS (16384)");
  if (p->routed_rows == 0) return PLK_OK;
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev != s->device)
    return plk_hip_set_error(PLK_E_ARGUMENT, "plk_mok_forward_static: the session's device must be the current one");
  unsigned char* const base = g_static_area[dev];  // resolved when the session was created on this device
  if (!base) return plk_hip_set_error(PLK_E_RESOURCE, "plk_mok_forward_static: the device's static area was not resolved");
  const uint64_t workspace = (uint64_t)(uintptr_t)(base + STATIC_WORKSPACE_OFFSET);

  // The launches' params images travel as the argument of a small kernel that stores them into the static area and
  // clears the workspace: no copy from host memory, no wait, and stream order puts it in front of the launches.
  const bool one = !s->two_launches && plk_mok::one_launch_ok(dims_of(p, 0), p->hidden_q);
  const int passes[2] = {one ? 0 : 1, 2};
  const int launches = one ? 1 : 2;
  StaticImages images;
  std::memset(&images, 0, sizeof images);
  for (int l = 0; l < launches; ++l)
    fill_image(s->link, p, passes[l], workspace, reinterpret_cast<unsigned char*>(images.words) + l * PLK_MOK_STATIC_IMAGE_BYTES);
  plk_mok_store_images<<<dim3(1), dim3(STATIC_IMAGE_WORDS), 0, (hipStream_t)stream>>>(
      images, reinterpret_cast<uint32_t*>(base), reinterpret_cast<uint32_t*>(base + STATIC_WORKSPACE_OFFSET), (int)words);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return plk_hip_set_error(PLK_E_RESOURCE, hipGetErrorString(e));
  s->used_static = true;
  for (int l = 0; l < launches && rc == PLK_OK; ++l)
    rc = launch_pass(s, p, passes[l], stream, (uint64_t)(uintptr_t)(base + l * PLK_MOK_STATIC_IMAGE_BYTES));
  return rc;
}

}  // extern "C"

// ---- MXFP8 block quantiser ---------------------------------------------------------------
// One wave per row slice: each lane owns 4 consecutive elements, 8 lanes one 32-block.
// OCP MX rule: scale byte = clamp(exponent_field(amax) - 8, 0, 254); elements are
// e4m3_rne(clamp(v * 2^(127 - byte), +-448)).
template <bool BF16>
__global__ void __launch_bounds__(256) mxfp8_quantize_kernel(const void* __restrict__ src, int64_t rows, int k,
                                                             uint8_t* __restrict__ dq, int ld_q,
                                                             uint8_t* __restrict__ dsc, int ld_sc) {
  const int blocks_per_row = k / 32;
  const int64_t nblocks = rows * (int64_t)blocks_per_row;
  const int sub = threadIdx.x & 7;
  for (int64_t blk = (int64_t)blockIdx.x * 32 + (threadIdx.x >> 3); blk < nblocks; blk += (int64_t)gridDim.x * 32) {
    const int64_t row = blk / blocks_per_row;
    const int cb = (int)(blk - row * blocks_per_row);
    const int64_t off = row * (int64_t)k + cb * 32 + sub * 4;
    float v[4];
    if (BF16) {
      const uint2 raw = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(src) + off);
      v[0] = __uint_as_float(raw.x << 16);
      v[1] = __uint_as_float(raw.x & 0xFFFF0000u);
      v[2] = __uint_as_float(raw.y << 16);
      v[3] = __uint_as_float(raw.y & 0xFFFF0000u);
    } else {
      const float4 raw = *reinterpret_cast<const float4*>(static_cast<const float*>(src) + off);
      v[0] = raw.x; v[1] = raw.y; v[2] = raw.z; v[3] = raw.w;
    }
    float amax = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
    amax = fmaxf(amax, __shfl_xor(amax, 1));
    amax = fmaxf(amax, __shfl_xor(amax, 2));
    amax = fmaxf(amax, __shfl_xor(amax, 4));
    // fmaxf drops a NaN operand: a NaN anywhere in the block is carried beside the maximum, and makes the block's
    // largest magnitude NaN (exponent field 255, like an infinity), as a maximum that propagates NaN would
    int has_nan = (v[0] != v[0]) | (v[1] != v[1]) | (v[2] != v[2]) | (v[3] != v[3]);
    has_nan |= __shfl_xor(has_nan, 1);
    has_nan |= __shfl_xor(has_nan, 2);
    has_nan |= __shfl_xor(has_nan, 4);
    int e = (has_nan ? 255 : (int)((__float_as_uint(amax) >> 23) & 0xFFu)) - 8;
    e = e < 0 ? 0 : e;
    const float inv = __uint_as_float((uint32_t)(254 - e) << 23);
    float s[4];
    for (int j = 0; j < 4; ++j) s[j] = fminf(fmaxf(v[j] * inv, -448.0f), 448.0f);  // (a NaN becomes -448 here: replaced below)
    int pk = 0;
    pk = __builtin_amdgcn_cvt_pk_fp8_f32(s[0], s[1], pk, false);
    pk = __builtin_amdgcn_cvt_pk_fp8_f32(s[2], s[3], pk, true);
    for (int j = 0; j < 4; ++j)  // a NaN element keeps its sign and becomes e4m3's NaN code
      if (v[j] != v[j]) pk = (pk & ~(0xFF << (8 * j))) | (int)((0x7Fu | ((__float_as_uint(v[j]) >> 24) & 0x80u)) << (8 * j));
    *reinterpret_cast<uint32_t*>(dq + row * (int64_t)ld_q + cb * 32 + sub * 4) = (uint32_t)pk;
    if (sub == 0) dsc[row * ld_sc + cb] = (uint8_t)e;
    // zero the pad bytes of the scale row once per row
    if (cb == 0 && sub == 1)
      for (int c = blocks_per_row; c < ld_sc; ++c) dsc[row * ld_sc + c] = 0;
  }
}

extern "C" int plk_mxfp8_quantize(uint64_t src, int src_is_bf16, int64_t rows, int32_t k, uint64_t dst_q,
                                  int32_t ld_q, uint64_t dst_sc, int32_t ld_sc, void* stream) {
  if (rows < 0 || k <= 0 || k % 32 || ld_sc * 32 < k || ld_q < k || ld_q % 4)
    return plk_hip_set_error(PLK_E_ARGUMENT,
                             "plk_mxfp8_quantize: k must be a positive multiple of 32 covered by ld_sc and ld_q");
  if (rows == 0) return PLK_OK;
  if (!src || !dst_q || !dst_sc) return plk_hip_set_error(PLK_E_ARGUMENT, "plk_mxfp8_quantize: null device address");
  const int64_t nblocks = rows * (int64_t)(k / 32);
  int64_t grid = (nblocks + 31) / 32;
  if (grid > 65536) grid = 65536;
  if (src_is_bf16)
    mxfp8_quantize_kernel<true><<<dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream>>>(
        (const void*)(uintptr_t)src, rows, k, (uint8_t*)(uintptr_t)dst_q, ld_q, (uint8_t*)(uintptr_t)dst_sc, ld_sc);
  else
    mxfp8_quantize_kernel<false><<<dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream>>>(
        (const void*)(uintptr_t)src, rows, k, (uint8_t*)(uintptr_t)dst_q, ld_q, (uint8_t*)(uintptr_t)dst_sc, ld_sc);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return plk_hip_set_error(PLK_E_RESOURCE, hipGetErrorString(e));
  return PLK_OK;
}

// ---- weight code layout conversion: row-major [rows, ld_q] -> K-tiled [K/64, rows, 64] ------
__global__ void __launch_bounds__(256) codes_to_k64_tiled_kernel(const uint8_t* __restrict__ src, int64_t rows, int ktiles,
                                                                  int64_t ld_q, uint8_t* __restrict__ dst) {
  const int64_t total = rows * (int64_t)ktiles * 4;  // 16-byte pieces
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int c = (int)(i & 3);
    const int64_t rt = i >> 2, kt = rt / rows, r = rt - kt * rows;
    const uint4 v = *reinterpret_cast<const uint4*>(src + r * ld_q + kt * 64 + c * 16);
    *reinterpret_cast<uint4*>(dst + i * 16) = v;
  }
}

extern "C" int plk_mxfp8_codes_to_k64_tiled(uint64_t src, int64_t rows, int32_t k, int64_t ld_q, uint64_t dst, void* stream) {
  if (rows < 0 || k <= 0 || k % 64 || ld_q < k || ld_q % 16 || (src & 15) || (dst & 15))
    return plk_hip_set_error(PLK_E_ARGUMENT, "plk_mxfp8_codes_to_k64_tiled: k must be a positive multiple of 64, ld_q a multiple of 16 not below k, addresses 16-byte aligned");
  if (rows == 0) return PLK_OK;
  if (!src || !dst) return plk_hip_set_error(PLK_E_ARGUMENT, "plk_mxfp8_codes_to_k64_tiled: null device address");
  int64_t grid = (rows * (k / 64) * 4 + 255) / 256;
  if (grid > 65536) grid = 65536;
  codes_to_k64_tiled_kernel<<<dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream>>>(
      (const uint8_t*)(uintptr_t)src, rows, k / 64, ld_q, (uint8_t*)(uintptr_t)dst);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return plk_hip_set_error(PLK_E_RESOURCE, hipGetErrorString(e));
  return PLK_OK;
}

// ---- scale layout conversion ---------------------------------------------------------------
__global__ void __launch_bounds__(256) scales_to_slot_major_kernel(const uint8_t* __restrict__ src, int64_t rows, int nblocks,
                                                                    int ld_sc, uint32_t* __restrict__ dst, int nslots) {
  const int64_t total = rows * (int64_t)nslots;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t s = i / rows, r = i - s * rows;
    uint32_t v = 0;
    for (int j = 0; j < 4; ++j) {
      const int b = (int)s * 4 + j;
      if (b < nblocks) v |= (uint32_t)src[r * ld_sc + b] << (8 * j);
    }
    dst[i] = v;
  }
}

extern "C" int plk_mxfp8_scales_to_slot_major(uint64_t src, int64_t rows, int32_t k, int32_t ld_sc, uint64_t dst,
                                              void* stream) {
  if (rows < 0 || k <= 0 || k % 32 || ld_sc * 32 < k)
    return plk_hip_set_error(PLK_E_ARGUMENT, "plk_mxfp8_scales_to_slot_major: k must be a positive multiple of 32 covered by ld_sc");
  if (rows == 0) return PLK_OK;
  if (!src || !dst) return plk_hip_set_error(PLK_E_ARGUMENT, "plk_mxfp8_scales_to_slot_major: null device address");
  const int nslots = (k + 127) / 128;
  int64_t grid = (rows * nslots + 255) / 256;
  if (grid > 65536) grid = 65536;
  scales_to_slot_major_kernel<<<dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream>>>(
      (const uint8_t*)(uintptr_t)src, rows, k / 32, ld_sc, (uint32_t*)(uintptr_t)dst, nslots);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return plk_hip_set_error(PLK_E_RESOURCE, hipGetErrorString(e));
  return PLK_OK;
}
