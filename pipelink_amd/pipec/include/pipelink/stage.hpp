// Authoring annotations of a PipeLink stage source for gfx950.
//
// In the device compile (hipcc) every PL_* macro expands to nothing.  With -DPIPELINK_EMIT the
// stage source is compiled as a host C++17 program instead (the device code is fenced off with
// `#ifndef PIPELINK_EMIT`): the macros become static registrations whose records -- evaluated
// with the real sizeof/alignof of the stage's own types -- are printed as one JSON object by
// pl::emit_main(), from which `pipec pack` assembles manifest.json.
//
// Same division of labour and macro names as the reference's
// pipec/src/pipec2/pack/include/pipelink/stage.hpp:1413-1477 (registrations) / :1488-1524
// (no-ops) and pack/runner.cpp; the record set is the subset the gfx950 backend consumes
// (stage, params, roles, exports, call seams, claims, counter and ring endpoints, variants,
// topology, facts).
#ifndef PIPELINK_STAGE_HPP
#define PIPELINK_STAGE_HPP

#ifdef PIPELINK_EMIT

#include <cstdio>
#include <initializer_list>
#include <string>
#include <utility>
#include <vector>

namespace pl {

inline std::vector<std::pair<std::string, std::string>>& registry() {
  static std::vector<std::pair<std::string, std::string>> r;  // (section, json object)
  return r;
}

inline std::string quote(const std::string& s) {
  std::string out = "\"";
  for (char c : s) {
    if (c == '"' || c == '\\') { out += '\\'; out += c; }
    else if (c == '\n') out += "\\n";
    else out += c;
  }
  return out + "\"";
}

struct reg {
  reg(const char* section, const std::string& json) { registry().emplace_back(section, json); }
};

inline std::string num(long long v) { return std::to_string(v); }

struct kv { const char* handle; long long value; };

inline std::string keyset(std::initializer_list<kv> key) {
  std::string out = "{";
  bool first = true;
  for (const kv& k : key) {
    if (!first) out += ",";
    first = false;
    out += quote(k.handle) + ":" + num(k.value);
  }
  return out + "}";
}

inline std::string strlist(std::initializer_list<const char*> items) {
  std::string out = "[";
  bool first = true;
  for (const char* s : items) {
    if (!first) out += ",";
    first = false;
    out += quote(s);
  }
  return out + "]";
}

inline int emit_main() {
  // {"section": [records...], ...} with sections in first-use order
  std::vector<std::string> sections;
  for (auto& e : registry()) {
    bool seen = false;
    for (auto& s : sections) seen = seen || s == e.first;
    if (!seen) sections.push_back(e.first);
  }
  std::printf("{");
  for (size_t i = 0; i < sections.size(); ++i) {
    std::printf("%s%s:[", i ? "," : "", quote(sections[i]).c_str());
    bool first = true;
    for (auto& e : registry())
      if (e.first == sections[i]) {
        std::printf("%s%s", first ? "" : ",", e.second.c_str());
        first = false;
      }
    std::printf("]");
  }
  std::printf("}\n");
  return 0;
}

}  // namespace pl

#define PL_CAT2(a, b) a##b
#define PL_CAT(a, b) PL_CAT2(a, b)
#define PL_REG(section, json) static const ::pl::reg PL_CAT(pl_reg_, __COUNTER__)(section, json)

#define PL_STAGE(id, version) PL_REG("stage", "{\"id\":" + ::pl::quote(id) + ",\"version\":" + ::pl::quote(version) + "}")
#define PL_PARAMS(T) \
  PL_REG("params", "{\"type\":" + ::pl::quote(#T) + ",\"bytes\":" + ::pl::num(sizeof(T)) + ",\"align\":" + ::pl::num(alignof(T)) + "}")
#define PL_NO_PARAMS() PL_REG("params", "{\"type\":\"void\",\"bytes\":0,\"align\":1}")
#define PL_ROLE(name, fn, warps) \
  PL_REG("roles", "{\"name\":" + ::pl::quote(#name) + ",\"entry\":" + ::pl::quote(#fn) + ",\"warps\":" + ::pl::num(warps) + "}")
// an exported device function: `decl` is its declaration text, identity-bearing for the call seam
#define PL_EXPORT(name, symbol, decl) \
  PL_REG("exports", "{\"name\":" + ::pl::quote(#name) + ",\"symbol\":" + ::pl::quote(#symbol) + ",\"decl\":" + ::pl::quote(decl) + "}")
// this stage calls export `export_name` of whoever consumes channel `channel` through the
// link-generated trampoline pipelink_call_<channel>; `decl` declares that trampoline
#define PL_CALL(channel, export_name, decl) \
  PL_REG("calls", "{\"channel\":" + ::pl::quote(#channel) + ",\"direction\":\"produce\",\"export\":" + ::pl::quote(export_name) + ",\"decl\":" + ::pl::quote(decl) + "}")
// this stage provides export `export_name` on channel `channel`
#define PL_SERVE(channel, export_name) \
  PL_REG("calls", "{\"channel\":" + ::pl::quote(#channel) + ",\"direction\":\"consume\",\"export\":" + ::pl::quote(export_name) + "}")
#define PL_CLAIM(handle, domain, extent, align, lifetime) \
  PL_REG("claims", "{\"handle\":" + ::pl::quote(handle) + ",\"domain\":" + ::pl::quote(domain) + ",\"extent\":{\"const\":" + ::pl::num(extent) + ",\"per\":{}},\"align\":" + ::pl::num(align) + ",\"lifetime\":" + ::pl::quote(lifetime) + "}")
// extent = base + per * value(depth_handle): an LDS ring whose depth is bound at link time
#define PL_CLAIM_RING(handle, domain, base, depth_handle, per, align, lifetime) \
  PL_REG("claims", "{\"handle\":" + ::pl::quote(handle) + ",\"domain\":" + ::pl::quote(domain) + ",\"extent\":{\"const\":" + ::pl::num(base) + ",\"per\":{" + ::pl::quote(depth_handle) + ":" + ::pl::num(per) + "}},\"align\":" + ::pl::num(align) + ",\"lifetime\":" + ::pl::quote(lifetime) + "}")
// the waves of role `role`: the handle's value is the index of the role's first wave in the workgroup
#define PL_CLAIM_WARPS(handle, role, warps) \
  PL_REG("claims", "{\"handle\":" + ::pl::quote(handle) + ",\"domain\":\"warp\",\"extent\":{\"const\":" + ::pl::num(warps) + ",\"per\":{}},\"align\":1,\"roles\":[" + ::pl::quote(#role) + "],\"lifetime\":\"kernel\"}")
#define PL_VARIANT(index, ...) \
  PL_REG("variants", "{\"index\":" + ::pl::num(index) + ",\"key\":" + ::pl::keyset(__VA_ARGS__) + "}")
#define PL_TOPOLOGY(persistent, scheduler) \
  PL_REG("topology", std::string("{\"persistent\":") + ((persistent) ? "true" : "false") + ",\"scheduler\":" + ::pl::quote(scheduler) + "}")
// a global-memory counter channel: release add on the producing side, acquire load on the other
#define PL_COUNTER(name, direction, slot_handle, exports) \
  PL_REG("counters", "{\"name\":" + ::pl::quote(#name) + ",\"direction\":" + ::pl::quote(direction) + ",\"slot\":" + ::pl::quote(slot_handle) + ",\"exports\":" + ::pl::strlist(exports) + "}")
// One end of an LDS ring with full / empty counters (protocol kind "mbarrier" in the manifest):
// `direction` "produce" or "consume"; the tile is one ring stage, rows x cols elements of `dtype`
// (`elem_bits` wide), `stride` bytes apart; `depth` is the depth handle; the full counters live in
// the slots of handle `full` and take `full_count` arrivals per fill from role `full_by`, the
// empty counters in `empty` with `empty_count` arrivals per drain from `empty_by` (counts are
// integers or expressions such as "warps(mma)"); `init_owner` is the role on whose behalf the
// dispatch kernel zeroes the counters.  Both ends must state the same thing.
#define PL_RING(name, direction, owner_role, dtype, elem_bits, rows, cols, depth, stride, full, full_count, full_by, empty, \
                empty_count, empty_by, init_owner)                                                                       \
  PL_REG("rings", "{\"name\":" + ::pl::quote(#name) + ",\"direction\":" + ::pl::quote(direction) + ",\"owner_role\":" +   \
                      ::pl::quote(#owner_role) + ",\"dtype\":" + ::pl::quote(dtype) + ",\"elem_bits\":" + ::pl::num(elem_bits) + \
                      ",\"rows\":" + ::pl::num(rows) + ",\"cols\":" + ::pl::num(cols) + ",\"depth\":" + ::pl::quote(depth) +   \
                      ",\"stride\":" + ::pl::num(stride) + ",\"full\":" + ::pl::quote(full) + ",\"full_count\":" +           \
                      ::pl::quote(full_count) + ",\"full_by\":" + ::pl::quote(#full_by) + ",\"empty\":" + ::pl::quote(empty) +  \
                      ",\"empty_count\":" + ::pl::quote(empty_count) + ",\"empty_by\":" + ::pl::quote(#empty_by) +            \
                      ",\"init_owner\":" + ::pl::quote(#init_owner) + "}")
// A tile this stage hands to whoever imports tensor `result`: `home` is "agpr", "vgpr" or "lds"; `layout`
// is "mfma32x32c" (registers: the frame handed over is rows * cols / 64 floats per lane) or "row_major"
// (lds: `row_pitch` bytes between rows of the wave's tile; 0 for register homes).  rows x cols is one
// participant's (one wave's) share.
#define PL_EXPORT_TENSOR(name, result, dtype, rows, cols, home, layout, row_pitch)                                         \
  PL_REG("tensor_exports", "{\"name\":" + ::pl::quote(#name) + ",\"result\":" + ::pl::quote(result) + ",\"dtype\":" +      \
                               ::pl::quote(dtype) + ",\"shape\":[" + ::pl::num(rows) + "," + ::pl::num(cols) + "],\"home\":" + \
                               ::pl::quote(home) + ",\"layout\":" + ::pl::quote(layout) + ",\"row_pitch_bytes\":" +        \
                               ::pl::num(row_pitch) + "}")
// This stage reads tensor `result` through the link-generated `fn(const void* source, float* dest)` (with
// `fn_ready()` before it and `fn_done()` after it), which delivers the elements in `layout`.
#define PL_IMPORT_TENSOR(name, fn, result, dtype, rows, cols, layout)                                                      \
  PL_REG("tensor_imports", "{\"name\":" + ::pl::quote(#name) + ",\"fn\":" + ::pl::quote(#fn) + ",\"result\":" +           \
                               ::pl::quote(result) + ",\"dtype\":" + ::pl::quote(dtype) + ",\"shape\":[" + ::pl::num(rows) + \
                               "," + ::pl::num(cols) + "],\"layout\":" + ::pl::quote(layout) + "}")
// a published geometry fact of this owner (reaches other owners only through the link)
// ---- host contract: what the broker needs to know to build this stage's params through a provider library
// (the reference's PL_HOST_GROUP / PL_HOST_ABI_* / PL_HOST_SCALARS / PL_HOST_CHANNEL, pack/include/pipelink/host.hpp).
// The link gathers these into link.json["host"]["groups"].
// the params group and the suffix of the provider's four entry points pipelink_params_{abi,query,build,release}_<suffix>
#define PL_HOST_GROUP(params_group, provider_suffix) \
  PL_REG("host_group", "{\"params_group\":" + ::pl::quote(params_group) + ",\"provider\":" + ::pl::quote(provider_suffix) + "}")
// an owner-local record type the provider reports: its id, and what this compiler makes of it
#define PL_HOST_ABI_TYPE(id, T) \
  PL_REG("host_types", "{\"id\":" + ::pl::num(id) + ",\"name\":" + ::pl::quote(#T) + ",\"bytes\":" + ::pl::num(sizeof(T)) + \
                           ",\"align\":" + ::pl::num(alignof(T)) + "}")
// a scalar of the shared scalar image: kind "i64" or "f64"
#define PL_HOST_SCALAR(id, name, kind) \
  PL_REG("host_scalars", "{\"id\":" + ::pl::num(id) + ",\"name\":" + ::pl::quote(name) + ",\"kind\":" + ::pl::quote(kind) + "}")
// a caller-owned tensor: channel id, caller's name, element bits, "read" or "write", extents as a comma-separated
// list of terms (an integer, a scalar name, floor(name,int) or ceil(name,int)), and whether the caller may leave it out
#define PL_HOST_CHANNEL(id, name, elem_bits, access, extents, optional)                                                      \
  PL_REG("host_channels", "{\"id\":" + ::pl::num(id) + ",\"name\":" + ::pl::quote(name) + ",\"elem_bits\":" +             \
                              ::pl::num(elem_bits) + ",\"access\":" + ::pl::quote(access) + ",\"extents\":" +              \
                              ::pl::quote(extents) + ",\"optional\":" + ((optional) ? "true" : "false") + "}")
#define PL_FACT(name, value) PL_REG("facts", "{\"name\":" + ::pl::quote(name) + ",\"value\":" + ::pl::num(value) + "}")
// a header whose declarations cross a call seam (task records, fragment types): its text
// travels in the package and the linker puts it in front of the generated trampolines
#define PL_PRELUDE(path) PL_REG("preludes", ::pl::quote(path))
// handles this stage reads through `extern "C" __device__ int <handle>()`
#define PL_USES(handle) PL_REG("uses", ::pl::quote(handle))

#define PL_EMIT_MAIN() \
  int main() { return ::pl::emit_main(); }

#else  // device compile: annotations vanish

#define PL_STAGE(id, version)
#define PL_PARAMS(T)
#define PL_NO_PARAMS()
#define PL_ROLE(name, fn, warps)
#define PL_EXPORT(name, symbol, decl)
#define PL_CALL(channel, export_name, decl)
#define PL_SERVE(channel, export_name)
#define PL_CLAIM(handle, domain, extent, align, lifetime)
#define PL_CLAIM_RING(handle, domain, base, depth_handle, per, align, lifetime)
#define PL_CLAIM_WARPS(handle, role, warps)
#define PL_VARIANT(index, ...)
#define PL_TOPOLOGY(persistent, scheduler)
#define PL_COUNTER(name, direction, slot_handle, exports)
#define PL_RING(name, direction, owner_role, dtype, elem_bits, rows, cols, depth, stride, full, full_count, full_by, empty, \
                empty_count, empty_by, init_owner)
#define PL_EXPORT_TENSOR(name, result, dtype, rows, cols, home, layout, row_pitch)
#define PL_IMPORT_TENSOR(name, fn, result, dtype, rows, cols, layout)
#define PL_HOST_GROUP(params_group, provider_suffix)
#define PL_HOST_ABI_TYPE(id, T)
#define PL_HOST_SCALAR(id, name, kind)
#define PL_HOST_CHANNEL(id, name, elem_bits, access, extents, optional)
#define PL_FACT(name, value)
#define PL_USES(handle)
#define PL_PRELUDE(path)
#define PL_EMIT_MAIN()

#endif
#endif
