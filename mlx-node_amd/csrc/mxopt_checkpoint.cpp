// Optimizer-state checkpoints as safetensors files: the format the reference's own writer produces
// (crates/mlx-core/src/utils/safetensors.rs:312-385: 8-byte little-endian header length, JSON
// header {name: {dtype, shape, data_offsets}, "__metadata__": {...}}, raw little-endian data).
// Moments are float32, so the reference writer's truncating bf16 encoder (:449-457) never applies.
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "mxopt_checkpoint_internal.h"

namespace mxopt {

namespace {

// ---- a JSON reader just large enough for a safetensors header ---------------------------
struct Json {
  enum Type { Null, Bool, Number, String, Array, Object } type = Null;
  double number = 0;
  std::string string;
  std::vector<Json> array;
  std::vector<std::pair<std::string, Json>> object;
  const Json* get(const std::string& key) const {
    for (const auto& kv : object)
      if (kv.first == key) return &kv.second;
    return nullptr;
  }
};

struct JsonReader {
  const char* p;
  const char* end;
  bool ok = true;
  void ws() { while (p < end && (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r')) ++p; }
  bool eat(char c) { ws(); if (p < end && *p == c) { ++p; return true; } return false; }
  std::string str() {
    std::string out;
    if (!eat('"')) { ok = false; return out; }
    while (p < end && *p != '"') {
      char c = *p++;
      if (c != '\\') { out.push_back(c); continue; }
      if (p >= end) { ok = false; return out; }
      char e = *p++;
      switch (e) {
        case 'n': out.push_back('\n'); break;
        case 't': out.push_back('\t'); break;
        case 'r': out.push_back('\r'); break;
        case 'b': out.push_back('\b'); break;
        case 'f': out.push_back('\f'); break;
        case 'u': {
          if (end - p < 4) { ok = false; return out; }
          unsigned cp = 0;
          for (int i = 0; i < 4; ++i) {
            char h = *p++;
            cp = cp * 16 + (h >= '0' && h <= '9' ? h - '0' : h >= 'a' && h <= 'f' ? h - 'a' + 10 :
                            h >= 'A' && h <= 'F' ? h - 'A' + 10 : (ok = false, 0));
          }
          if (cp < 0x80) out.push_back((char)cp);
          else if (cp < 0x800) { out.push_back((char)(0xC0 | (cp >> 6))); out.push_back((char)(0x80 | (cp & 0x3F))); }
          else { out.push_back((char)(0xE0 | (cp >> 12))); out.push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
                 out.push_back((char)(0x80 | (cp & 0x3F))); }
          break;
        }
        default: out.push_back(e);  // \" \\ \/
      }
    }
    if (p >= end) { ok = false; return out; }
    ++p;
    return out;
  }
  Json value(int depth = 0) {
    Json v;
    ws();
    if (p >= end || depth > 16) { ok = false; return v; }
    if (*p == '{') {
      ++p;
      v.type = Json::Object;
      if (eat('}')) return v;
      do {
        std::string k = str();
        if (!ok || !eat(':')) { ok = false; return v; }
        v.object.emplace_back(std::move(k), value(depth + 1));
      } while (ok && eat(','));
      if (!eat('}')) ok = false;
    } else if (*p == '[') {
      ++p;
      v.type = Json::Array;
      if (eat(']')) return v;
      do v.array.push_back(value(depth + 1)); while (ok && eat(','));
      if (!eat(']')) ok = false;
    } else if (*p == '"') {
      v.type = Json::String;
      v.string = str();
    } else if (end - p >= 4 && !std::strncmp(p, "true", 4)) { v.type = Json::Bool; v.number = 1; p += 4; }
    else if (end - p >= 5 && !std::strncmp(p, "false", 5)) { v.type = Json::Bool; p += 5; }
    else if (end - p >= 4 && !std::strncmp(p, "null", 4)) { p += 4; }
    else {
      char* stop = nullptr;
      std::string tmp(p, std::min<size_t>(end - p, 40));
      v.number = std::strtod(tmp.c_str(), &stop);
      if (stop == tmp.c_str()) { ok = false; return v; }
      v.type = Json::Number;
      p += stop - tmp.c_str();
    }
    return v;
  }
};

std::string json_escape(const std::string& s) {
  std::string out;
  for (unsigned char c : s) {
    if (c == '"' || c == '\\') { out.push_back('\\'); out.push_back((char)c); }
    else if (c < 0x20) { char buf[8]; std::snprintf(buf, sizeof buf, "\\u%04x", c); out += buf; }
    else out.push_back((char)c);
  }
  return out;
}

constexpr size_t kStageBytes = 32u << 20;

struct Staging {  // pinned bounce buffer for the device <-> file copies
  void* host = nullptr;
  ~Staging() { if (host) (void)hipHostFree(host); }
  int ensure(mxopt_ctx* ctx) {
    if (!host) HIP_TRY(ctx, hipHostMalloc(&host, kStageBytes, hipHostMallocDefault));
    return MXOPT_OK;
  }
};

struct FileCloser {
  FILE* f;
  ~FileCloser() { if (f) std::fclose(f); }
};

}  // namespace

int save_state_file(mxopt_ctx* ctx, const char* path, const char* optimizer, int64_t step,
                    const std::vector<CheckpointTensor>& tensors) {
  if (!path) return fail(ctx, MXOPT_ERR_INVALID_ARG, "save_file: path is NULL");
  std::vector<const CheckpointTensor*> order;
  for (const auto& t : tensors) order.push_back(&t);
  std::sort(order.begin(), order.end(),
            [](const CheckpointTensor* a, const CheckpointTensor* b) { return a->key < b->key; });  // as :325-327
  std::string header = "{";
  uint64_t offset = 0;
  for (const CheckpointTensor* t : order) {
    const uint64_t bytes = t->n * sizeof(float);
    header += "\"" + json_escape(t->key) + "\":{\"dtype\":\"F32\",\"shape\":[" + std::to_string(t->n) +
              "],\"data_offsets\":[" + std::to_string(offset) + "," + std::to_string(offset + bytes) + "]},";
    offset += bytes;
  }
  header += "\"__metadata__\":{\"format\":\"mxopt-optimizer-state\",\"optimizer\":\"" + std::string(optimizer) +
            "\",\"step\":\"" + std::to_string(step) + "\"}}";
  while (header.size() % 8) header.push_back(' ');

  const std::string tmp = std::string(path) + ".tmp";
  FileCloser file{std::fopen(tmp.c_str(), "wb")};
  if (!file.f) return fail(ctx, MXOPT_ERR_FAILURE, "save_file: cannot create " + tmp);
  const uint64_t hlen = header.size();
  unsigned char le[8];
  for (int i = 0; i < 8; ++i) le[i] = (unsigned char)(hlen >> (8 * i));
  bool ok = std::fwrite(le, 1, 8, file.f) == 8 && std::fwrite(header.data(), 1, header.size(), file.f) == header.size();

  DeviceGuard guard(ctx->device);
  Staging stage;
  // Any failure from here on closes and removes the half-written temporary file.
  auto abandon = [&](int code) {
    if (file.f) { std::fclose(file.f); file.f = nullptr; }
    std::remove(tmp.c_str());
    return code;
  };
  int rc = stage.ensure(ctx);
  if (rc) return abandon(rc);
  for (const CheckpointTensor* t : order) {
    const char* src = (const char*)t->device;
    uint64_t left = t->n * sizeof(float);
    while (ok && left) {
      const size_t now = (size_t)std::min<uint64_t>(left, kStageBytes);
      hipError_t err = hipMemcpyAsync(stage.host, src, now, hipMemcpyDeviceToHost, ctx->stream);
      if (err == hipSuccess) err = hipStreamSynchronize(ctx->stream);
      if (err != hipSuccess) return abandon(hip_fail(ctx, err, "save_file: copying state to the host"));
      ok = std::fwrite(stage.host, 1, now, file.f) == now;
      src += now;
      left -= now;
    }
  }
  ok = ok && std::fflush(file.f) == 0;
  std::fclose(file.f);
  file.f = nullptr;
  if (!ok) {
    std::remove(tmp.c_str());
    return fail(ctx, MXOPT_ERR_FAILURE, std::string("save_file: write to ") + tmp + " failed");
  }
  if (std::rename(tmp.c_str(), path) != 0) {
    std::remove(tmp.c_str());
    return fail(ctx, MXOPT_ERR_FAILURE, std::string("save_file: cannot rename to ") + path);
  }
  return MXOPT_OK;
}

namespace {

struct Entry { std::string key; uint64_t begin, end; };

// Reads and validates the header: format tag, optimizer kind, step, and every tensor's byte range
// against the size of the file.  No device involved.
int read_header(mxopt_ctx* ctx, FILE* f, std::string* optimizer, int64_t* step,
                std::vector<Entry>* entries, uint64_t* data_start) {
  unsigned char le[8];
  if (std::fread(le, 1, 8, f) != 8) return fail(ctx, MXOPT_ERR_FAILURE, "load_file: file is too short");
  uint64_t hlen = 0;
  for (int i = 0; i < 8; ++i) hlen |= (uint64_t)le[i] << (8 * i);
  if (hlen < 2 || hlen > (256u << 20)) return fail(ctx, MXOPT_ERR_FAILURE, "load_file: implausible header length");
  std::string header(hlen, '\0');
  if (std::fread(&header[0], 1, hlen, f) != hlen) return fail(ctx, MXOPT_ERR_FAILURE, "load_file: truncated header");
  JsonReader rd{header.data(), header.data() + header.size()};
  const Json root = rd.value();
  if (!rd.ok || root.type != Json::Object) return fail(ctx, MXOPT_ERR_FAILURE, "load_file: header is not a JSON object");
  const Json* meta = root.get("__metadata__");
  const Json* fmt = meta && meta->type == Json::Object ? meta->get("format") : nullptr;
  if (!fmt || fmt->string != "mxopt-optimizer-state")
    return fail(ctx, MXOPT_ERR_INVALID_ARG, "load_file: not an optimizer-state checkpoint");
  const Json* kind = meta->get("optimizer");
  *optimizer = kind ? kind->string : "";
  for (char ch : *optimizer)  // the name goes back to the caller as a C string: plain identifiers only
    if (!((ch >= 'a' && ch <= 'z') || (ch >= 'A' && ch <= 'Z') || (ch >= '0' && ch <= '9') || ch == '_' || ch == '-'))
      return fail(ctx, MXOPT_ERR_INVALID_ARG, "load_file: the optimizer name in the metadata is not a plain identifier");
  const Json* st = meta->get("step");
  if (step) *step = st ? std::strtoll(st->string.c_str(), nullptr, 10) : 0;
  if (std::fseek(f, 0, SEEK_END) != 0) return fail(ctx, MXOPT_ERR_FAILURE, "load_file: seek failed");
  const long size = std::ftell(f);
  if (size < 0 || (uint64_t)size < 8 + hlen) return fail(ctx, MXOPT_ERR_FAILURE, "load_file: truncated header");
  const uint64_t data_bytes = (uint64_t)size - 8 - hlen;  // the file size bounds every offset
  *data_start = 8 + hlen;
  for (const auto& kv : root.object) {
    if (kv.first == "__metadata__") continue;
    const Json* dt = kv.second.type == Json::Object ? kv.second.get("dtype") : nullptr;
    const Json* off = kv.second.type == Json::Object ? kv.second.get("data_offsets") : nullptr;
    if (!dt || !off || off->array.size() != 2 || off->array[0].type != Json::Number || off->array[1].type != Json::Number)
      return fail(ctx, MXOPT_ERR_FAILURE, "load_file: malformed entry '" + kv.first + "'");
    if (dt->string != "F32") return fail(ctx, MXOPT_ERR_INVALID_ARG, "load_file: '" + kv.first + "' is not float32");
    const double da = off->array[0].number, db = off->array[1].number;
    if (!(da >= 0) || !(db >= da) || db > (double)data_bytes)
      return fail(ctx, MXOPT_ERR_FAILURE, "load_file: '" + kv.first + "' has offsets outside the file");
    const uint64_t a = (uint64_t)da, b = (uint64_t)db;
    if ((b - a) % 4) return fail(ctx, MXOPT_ERR_FAILURE, "load_file: '" + kv.first + "' is not a whole number of floats");
    entries->push_back({kv.first, a, b});
  }
  return MXOPT_OK;
}

}  // namespace

int inspect_state_file(const char* path, std::string* optimizer, int64_t* step, uint64_t* tensors, uint64_t* elements) {
  if (!path) return fail(nullptr, MXOPT_ERR_INVALID_ARG, "checkpoint_inspect: path is NULL");
  FileCloser file{std::fopen(path, "rb")};
  if (!file.f) return fail(nullptr, MXOPT_ERR_FAILURE, std::string("load_file: cannot open ") + path);
  std::vector<Entry> entries;
  uint64_t data_start = 0;
  int rc = read_header(nullptr, file.f, optimizer, step, &entries, &data_start);
  if (rc) return rc;
  if (tensors) *tensors = entries.size();
  if (elements) {
    *elements = 0;
    for (const Entry& e : entries) *elements += (e.end - e.begin) / 4;
  }
  return MXOPT_OK;
}

int load_state_file(mxopt_ctx* ctx, const char* path, const char* optimizer, int64_t* step,
                    const std::function<int(const std::string& key, uint64_t n, float** device)>& place) {
  if (!path) return fail(ctx, MXOPT_ERR_INVALID_ARG, "load_file: path is NULL");
  FileCloser file{std::fopen(path, "rb")};
  if (!file.f) return fail(ctx, MXOPT_ERR_FAILURE, std::string("load_file: cannot open ") + path);
  std::vector<Entry> entries;
  std::string kind;
  uint64_t data_start = 0;
  int rc = read_header(ctx, file.f, &kind, step, &entries, &data_start);
  if (rc) return rc;
  if (kind != optimizer)
    return fail(ctx, MXOPT_ERR_INVALID_ARG, std::string("load_file: checkpoint is for optimizer '") + kind +
                "', this one is '" + optimizer + "'");
  DeviceGuard guard(ctx->device);
  Staging stage;
  if ((rc = stage.ensure(ctx))) return rc;
  for (const Entry& entry : entries) {
    const uint64_t a = entry.begin, b = entry.end;
    const uint64_t n = (b - a) / 4;
    float* dst = nullptr;
    if ((rc = place(entry.key, n, &dst))) return rc;
    if (!dst || !n) continue;
    if (std::fseek(file.f, (long)(data_start + a), SEEK_SET) != 0) return fail(ctx, MXOPT_ERR_FAILURE, "load_file: seek failed");
    char* d = (char*)dst;
    uint64_t left = b - a;
    while (left) {
      const size_t now = (size_t)std::min<uint64_t>(left, kStageBytes);
      if (std::fread(stage.host, 1, now, file.f) != now) return fail(ctx, MXOPT_ERR_FAILURE, "load_file: truncated data");
      HIP_TRY(ctx, hipMemcpyAsync(d, stage.host, now, hipMemcpyHostToDevice, ctx->stream));
      HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
      d += now;
      left -= now;
    }
  }
  return MXOPT_OK;
}

}  // namespace mxopt
