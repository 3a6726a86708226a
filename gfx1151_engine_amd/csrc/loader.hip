// Checkpoint files -> HBM: reads the MoE tensors of a .hgn (HGN1) or GGUF file and registers them in a
// context.  Host code only: the file is mapped read-only, every tensor of the path is copied to
// device memory once (one allocation per tensor, bytes unchanged) and handed to moe_set_*.
// On the reference's APU the experts are read in place from registered host memory; here they
// are resident in HBM.
// (reference: src/hgn.h:48-76,295-363 header / record layout and map_file; src/gguf.h:225-314 GGUF
//  header, key-value section, tensor infos; tensor names src/gpu/parts/40_model.inc:1808-1857,
//  src/gpu/parts/30_host_util.inc:384-412, src/gguf_map.h:210-214)
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstring>
#include <memory>
#include <new>
#include <thread>
#include <string>
#include <unordered_map>
#include <vector>

#include "common.h"

namespace {

struct FTensor {
  int dtype = 0;  // hgn dtype or ggml type
  uint32_t nd = 0;
  uint64_t dims[4] = {1, 1, 1, 1};  // hgn: outermost first (cols last); gguf: ne[] (cols first)
  const uint8_t* data = nullptr;
  uint64_t nbytes = 0;
};

#pragma pack(push, 1)
struct HgnHeader {  // src/hgn.h:48-54
  char magic[4];
  uint32_t version, tensor_count, reserved;
  uint64_t records_offset, data_offset, file_size;
  char model_name[64];
};
struct HgnRecord {  // src/hgn.h:55-60
  char name[96];
  uint32_t dtype, ndims;
  uint64_t dims[4];
  uint64_t data_offset, data_size, extra;
};
#pragma pack(pop)
static_assert(sizeof(HgnHeader) == 104 && sizeof(HgnRecord) == 160, "HGN1 on-disk structs");

// ggml tensor types this reader can size: {type id, elements per block, bytes per block}, ordered by id
// (the constants are ggml's on-disk format; src/gguf.h:42-64 lists the same ones)
struct GgmlGeom { uint16_t type, elems, bytes; };
constexpr GgmlGeom kGgmlGeom[] = {
    {0, 1, 4},      {1, 1, 2},      {2, 32, 18},    {3, 32, 20},    {6, 32, 22},    {7, 32, 24},   {8, 32, 34},
    {10, 256, 84},  {11, 256, 110}, {12, 256, 144}, {13, 256, 176}, {14, 256, 210}, {20, 32, 18},  {23, 256, 136},
    {24, 1, 1},     {25, 1, 2},     {26, 1, 4},     {27, 1, 8},     {28, 1, 8},     {30, 1, 2}};
bool ggml_block(uint32_t t, uint32_t& be, uint32_t& bb) {
  for (const GgmlGeom& g : kGgmlGeom)
    if (g.type == t) {
      be = g.elems;
      bb = g.bytes;
      return true;
    }
  be = bb = 0;
  return false;
}

struct Cur {  // bounds-checked little-endian reader over the mapped header
  const uint8_t *p, *end;
  bool ok = true;
  template <class T>
  T get() {
    T v{};
    if (!ok || (size_t)(end - p) < sizeof(T)) { ok = false; return v; }
    memcpy(&v, p, sizeof(T));
    p += sizeof(T);
    return v;
  }
  std::string str() {
    const uint64_t n = get<uint64_t>();
    if (!ok || (uint64_t)(end - p) < n) { ok = false; return {}; }
    std::string s((const char*)p, (size_t)n);
    p += n;
    return s;
  }
  void skip(uint64_t n) {
    if (!ok || (uint64_t)(end - p) < n) { ok = false; return; }
    p += n;
  }
};

// size of a scalar GGUF value type, 0 for string (8) / array (9) / unknown
uint32_t gguf_scalar_bytes(uint32_t t) {
  switch (t) {
    case 0: case 1: case 7: return 1;
    case 2: case 3: return 2;
    case 4: case 5: case 6: return 4;
    case 10: case 11: case 12: return 8;
    default: return 0;
  }
}

}  // namespace

struct FMap {  // one mapped file: the base file, a GGUF shard or an .hgn overlay
  int fd = -1;
  const uint8_t* base = nullptr;
  size_t len = 0;
  dev_t dev = 0;
  ino_t ino = 0;
};

struct moe_file {
  int format = 0;
  std::vector<FMap> maps;
  std::unordered_map<std::string, FTensor> idx;
  std::unordered_map<std::string, int64_t> kv_int;  // GGUF integer metadata
  bool gguf_keep_f32 = false;  // MOE_FILE_OPT_GGUF_F32_ROUTER
};

namespace {
struct Stager;
}
struct moe_weights {
  std::vector<void*> dev;
  uint64_t bytes = 0;
  std::shared_ptr<Stager> stager;  // pinned staging buffers, kept for the duration of one moe_load_layers call
};

// hgn v2 dtypes (ht, i4r, q6g64): an overlay must not replace tensors stored that way (src/hgn.h:292)
static bool hgn_v2_dtype(int dt) { return dt == 16 || dt == 23 || dt == 24; }

// Indexes the tensors of one mapped HGN1 file.  Base file: the first record of a name wins.  Overlay
// (hgn::Checkpoint::add_overlay, src/hgn.h:108-121,348-362): its tensors replace those of the same name, unless
// one of them would replace an hgn v2 tensor -- then the whole file is left out (*skipped = true).
static int parse_hgn(moe_file* f, const FMap& m, bool overlay, bool* skipped) {
  if (m.len < sizeof(HgnHeader)) return MOE_E_INVALID;
  HgnHeader h;
  memcpy(&h, m.base, sizeof h);
  if (memcmp(h.magic, "HGN1", 4) != 0) return MOE_E_UNSUPPORTED;
  if (h.file_size != m.len) return MOE_E_INVALID;  // the reference rejects a size mismatch too
  if (h.records_offset > m.len || (uint64_t)h.tensor_count * sizeof(HgnRecord) > m.len - h.records_offset)
    return MOE_E_INVALID;
  std::vector<std::pair<std::string, FTensor>> ts;
  ts.reserve(h.tensor_count);
  for (uint32_t i = 0; i < h.tensor_count; i++) {
    HgnRecord r;
    memcpy(&r, m.base + h.records_offset + (uint64_t)i * sizeof r, sizeof r);
    if (r.data_offset > m.len || r.data_size > m.len - r.data_offset || r.ndims > 4) return MOE_E_INVALID;
    FTensor t;
    t.dtype = (int)r.dtype;
    t.nd = r.ndims;
    for (int k = 0; k < 4; k++) t.dims[k] = k < (int)r.ndims ? r.dims[k] : 1;
    t.data = m.base + r.data_offset;
    t.nbytes = r.data_size;
    std::string name(r.name, strnlen(r.name, sizeof r.name));
    if (overlay) {
      auto it = f->idx.find(name);
      if (it != f->idx.end() && hgn_v2_dtype(it->second.dtype)) {
        *skipped = true;
        return MOE_OK;
      }
    }
    ts.emplace_back(std::move(name), t);
  }
  for (auto& nt : ts) {
    if (overlay) f->idx[nt.first] = nt.second;
    else f->idx.emplace(nt.first, nt.second);  // first record of a name wins
  }
  return MOE_OK;
}

// Indexes one GGUF file or shard (src/gguf.h:230-314): metadata of the first shard wins, later shards only add
// keys it does not have; general.alignment is read from the merged metadata.
static int parse_gguf(moe_file* f, const FMap& m, int shard) {
  if (m.len < 8 || memcmp(m.base, "GGUF", 4) != 0) return MOE_E_UNSUPPORTED;
  Cur c{m.base + 4, m.base + m.len};
  const uint32_t ver = c.get<uint32_t>();
  if (!c.ok || ver < 2) return MOE_E_UNSUPPORTED;
  const uint64_t nt = c.get<uint64_t>(), nkv = c.get<uint64_t>();
  uint64_t align = 32;
  for (uint64_t i = 0; i < nkv && c.ok; i++) {
    const std::string key = c.str();
    uint32_t t = c.get<uint32_t>();
    if (t == 9) {  // array: element type, count, elements
      const uint32_t et = c.get<uint32_t>();
      const uint64_t n = c.get<uint64_t>();
      if (et == 8) {
        for (uint64_t j = 0; j < n && c.ok; j++) (void)c.str();
      } else {
        const uint32_t sz = gguf_scalar_bytes(et);
        uint64_t bytes;
        if (!sz || __builtin_mul_overflow(n, (uint64_t)sz, &bytes)) return MOE_E_INVALID;
        c.skip(bytes);
      }
    } else if (t == 8) {
      (void)c.str();
    } else {
      const uint32_t sz = gguf_scalar_bytes(t);
      if (!sz) return MOE_E_INVALID;
      int64_t v = 0;
      bool is_int = true;
      switch (t) {
        case 0: v = c.get<uint8_t>(); break;
        case 1: v = c.get<int8_t>(); break;
        case 2: v = c.get<uint16_t>(); break;
        case 3: v = c.get<int16_t>(); break;
        case 4: v = c.get<uint32_t>(); break;
        case 5: v = c.get<int32_t>(); break;
        case 7: v = c.get<uint8_t>(); break;
        case 10: v = (int64_t)c.get<uint64_t>(); break;
        case 11: v = c.get<int64_t>(); break;
        default: c.skip(sz); is_int = false; break;  // floats
      }
      if (is_int && (shard == 0 || !f->kv_int.count(key))) f->kv_int[key] = v;
    }
  }
  if (!c.ok) return MOE_E_INVALID;
  if (auto it = f->kv_int.find("general.alignment"); it != f->kv_int.end()) {
    // a power of two of at most 4096 (ggml's default is 32): anything else is a corrupt or crafted header
    const int64_t a = it->second;
    if (a < 1 || a > 4096 || (a & (a - 1))) return MOE_E_INVALID;
    align = (uint64_t)a;
  }
  struct Pending { std::string name; FTensor t; uint64_t off; };
  std::vector<Pending> ts;
  for (uint64_t i = 0; i < nt && c.ok; i++) {
    Pending p;
    p.name = c.str();
    p.t.nd = c.get<uint32_t>();
    if (p.t.nd > 4) return MOE_E_INVALID;
    for (uint32_t k = 0; k < p.t.nd; k++) p.t.dims[k] = c.get<uint64_t>();
    p.t.dtype = (int)c.get<uint32_t>();
    p.off = c.get<uint64_t>();
    ts.push_back(std::move(p));
  }
  if (!c.ok) return MOE_E_INVALID;
  const uint64_t hdr = (uint64_t)(c.p - m.base);  // <= file length; align <= 4096: no wrap-around below
  const uint64_t data0 = (hdr + align - 1) & ~(align - 1);
  for (auto& p : ts) {
    uint32_t be, bb;
    if (!ggml_block((uint32_t)p.t.dtype, be, bb)) return MOE_E_UNSUPPORTED;
    // element count without wrap-around: a crafted file must not get a small byte size for huge dims
    uint64_t numel = 1;
    for (int k = 0; k < 4; k++)
      if (__builtin_mul_overflow(numel, p.t.dims[k], &numel)) return MOE_E_INVALID;
    if (p.t.dims[0] % be) return MOE_E_INVALID;
    if (__builtin_mul_overflow(numel / be, (uint64_t)bb, &p.t.nbytes)) return MOE_E_INVALID;
    uint64_t off;
    if (__builtin_add_overflow(data0, p.off, &off)) return MOE_E_INVALID;  // an offset that wraps around to the header
    if (off > m.len || p.t.nbytes > m.len - off) return MOE_E_INVALID;
    p.t.data = m.base + off;
    if (!f->idx.emplace(p.name, p.t).second) return MOE_E_INVALID;  // duplicate name
  }
  return MOE_OK;
}

MOE_API int moe_file_close(moe_file* f) {
  if (!f) return MOE_OK;
  for (FMap& m : f->maps) {
    if (m.base) munmap((void*)m.base, m.len);
    if (m.fd >= 0) close(m.fd);
  }
  delete f;
  return MOE_OK;
}

// maps `path` read-only and appends it to f->maps
static int map_one(moe_file* f, const char* path) {
  FMap m;
  m.fd = open(path, O_RDONLY | O_CLOEXEC);
  struct stat st;
  if (m.fd < 0 || fstat(m.fd, &st) < 0 || st.st_size < 8) {
    if (m.fd >= 0) close(m.fd);
    return MOE_E_INVALID;
  }
  m.len = (size_t)st.st_size;
  m.dev = st.st_dev;
  m.ino = st.st_ino;
  void* p = mmap(nullptr, m.len, PROT_READ, MAP_PRIVATE, m.fd, 0);
  if (p == MAP_FAILED) {
    close(m.fd);
    return MOE_E_STATE;
  }
  m.base = (const uint8_t*)p;
  f->maps.push_back(m);
  return MOE_OK;
}

// "<stem>-<5 digits>-of-<5 digits>.gguf": the reference opens all n shards when it is given any one of them
// (src/gguf.h:133-150).  Returns n (0: not a shard name) and the stem with its trailing '-'.
static int gguf_shard_count(const std::string& path, std::string* stem) {
  const size_t p = path.rfind("-of-");
  if (p == std::string::npos || p < 6 || path.size() != p + 4 + 5 + 5 || path.compare(path.size() - 5, 5, ".gguf") != 0)
    return 0;
  for (size_t i = p - 5; i < p; i++)
    if (path[i] < '0' || path[i] > '9') return 0;
  if (path[p - 6] != '-') return 0;
  int n = 0;
  for (size_t i = p + 4; i < p + 9; i++) {
    if (path[i] < '0' || path[i] > '9') return 0;
    n = n * 10 + (path[i] - '0');
  }
  *stem = path.substr(0, p - 5);
  return n;
}

MOE_API int moe_file_open(const char* path, moe_file** out) {
  if (!path || !out) return MOE_E_INVALID;
  moe_file* f = new (std::nothrow) moe_file();
  if (!f) return MOE_E_STATE;
  int rc = map_one(f, path);
  if (rc == MOE_OK) {
    const FMap& m0 = f->maps[0];
    if (memcmp(m0.base, "HGN1", 4) == 0) {
      f->format = MOE_FILE_HGN;
      bool skipped = false;
      rc = parse_hgn(f, m0, false, &skipped);
    } else if (memcmp(m0.base, "GGUF", 4) == 0) {
      f->format = MOE_FILE_GGUF;
      std::string stem;
      const int n = gguf_shard_count(path, &stem);
      if (n > 0) {  // a sharded model: every shard, in order (the mapping made above is dropped for shard 1's)
        munmap((void*)m0.base, m0.len);
        close(m0.fd);
        f->maps.clear();
        for (int i = 1; i <= n && rc == MOE_OK; i++) {
          char buf[32];
          snprintf(buf, sizeof buf, "%05d-of-%05d.gguf", i, n);
          rc = map_one(f, (stem + buf).c_str());
          if (rc == MOE_OK) rc = parse_gguf(f, f->maps.back(), i - 1);
        }
      } else {
        rc = parse_gguf(f, m0, 0);
      }
    } else {
      rc = MOE_E_UNSUPPORTED;
    }
  }
  if (rc != MOE_OK) {
    moe_file_close(f);
    return rc;
  }
  *out = f;
  return MOE_OK;
}

MOE_API int moe_file_add_overlay(moe_file* f, const char* path) {
  if (!f || !path) return MOE_E_INVALID;
  if (f->format != MOE_FILE_HGN) return MOE_E_UNSUPPORTED;
  int rc = map_one(f, path);
  if (rc != MOE_OK) return rc;
  auto drop_last = [&]() {
    FMap& m = f->maps.back();
    munmap((void*)m.base, m.len);
    close(m.fd);
    f->maps.pop_back();
  };
  const FMap& m = f->maps.back();
  for (size_t i = 0; i + 1 < f->maps.size(); i++)
    if (f->maps[i].dev == m.dev && f->maps[i].ino == m.ino) {  // already mapped (the reference compares paths)
      drop_last();
      return MOE_E_STATE;
    }
  bool skipped = false;
  rc = parse_hgn(f, m, true, &skipped);
  if (rc != MOE_OK || skipped) {
    drop_last();
    return rc != MOE_OK ? rc : MOE_E_STATE;
  }
  return MOE_OK;
}

MOE_API int moe_file_format(const moe_file* f) { return f ? f->format : 0; }
MOE_API int64_t moe_file_tensor_count(const moe_file* f) { return f ? (int64_t)f->idx.size() : 0; }

MOE_API int moe_file_find(const moe_file* f, const char* name, moe_tensor_info* out) {
  if (!f || !name || !out) return MOE_E_INVALID;
  auto it = f->idx.find(name);
  if (it == f->idx.end()) return MOE_E_STATE;
  out->dtype = it->second.dtype;
  out->ndims = it->second.nd;
  for (int k = 0; k < 4; k++) out->dims[k] = it->second.dims[k];
  out->data = it->second.data;
  out->nbytes = it->second.nbytes;
  return MOE_OK;
}

namespace {

const FTensor* find(const moe_file* f, const char* fmt, int layer) {
  char n[128];
  snprintf(n, sizeof n, fmt, layer);
  auto it = f->idx.find(n);
  return it == f->idx.end() ? nullptr : &it->second;
}

// rows x cols of a matrix tensor: hgn dims are outermost first (3-D fused experts flatten to
// [E*rows, cols], src/hgn.h:7-8), gguf ne[] is innermost first
bool matrix_shape(int format, const FTensor& t, uint64_t& rows, uint64_t& cols) {
  rows = 1;
  if (format == MOE_FILE_HGN) {
    cols = t.dims[t.nd ? t.nd - 1 : 0];
    for (uint32_t k = 0; k + 1 < t.nd; k++)
      if (__builtin_mul_overflow(rows, t.dims[k], &rows)) return false;
  } else {
    cols = t.dims[0];
    for (int k = 1; k < 4; k++)
      if (__builtin_mul_overflow(rows, t.dims[k], &rows)) return false;
  }
  return true;
}

}  // namespace

// Shapes of the path read off the tensors of layer `layer`: d, mid, experts; layers = the number of
// consecutive layers from `layer` on that carry the expert tensors.  topk is not stored in a .hgn
// file; GGUF files carry "<arch>.expert_used_count".  max_tokens / id_stride are left untouched.
MOE_API int moe_file_config(const moe_file* f, int layer, moe_config* cfg) {
  if (!f || !cfg || layer < 0) return MOE_E_INVALID;
  const bool hgn = f->format == MOE_FILE_HGN;
  const char* dn_name = hgn ? "layers.%d.mlp.experts.down_proj.weight" : "blk.%d.ffn_down_exps.weight";
  const FTensor* dn = find(f, dn_name, layer);
  if (!dn) return MOE_E_STATE;
  if (hgn) {
    // [E, d, mid] (or flat [E*d, mid] with the router giving E)
    const FTensor* rt = find(f, "layers.%d.mlp.gate.weight", layer);
    if (!rt || rt->nd != 2) return MOE_E_STATE;
    uint64_t rows, cols;
    if (!matrix_shape(f->format, *dn, rows, cols) || rt->dims[0] > (1u << 20) || rt->dims[1] > (1u << 24) ||
        cols > (1u << 24))
      return MOE_E_INVALID;
    cfg->experts = (int)rt->dims[0];
    cfg->d = (int)rt->dims[1];
    cfg->mid = (int)cols;
    if (rows != (uint64_t)cfg->experts * cfg->d) return MOE_E_INVALID;
  } else {
    if (dn->nd != 3 || dn->dims[0] > (1u << 24) || dn->dims[1] > (1u << 24) || dn->dims[2] > (1u << 20))
      return MOE_E_INVALID;
    cfg->mid = (int)dn->dims[0];
    cfg->d = (int)dn->dims[1];
    cfg->experts = (int)dn->dims[2];
    for (auto& kv : f->kv_int)
      if (kv.first.size() > 18 && kv.first.compare(kv.first.size() - 18, 18, ".expert_used_count") == 0)
        cfg->topk = (int)kv.second;
  }
  int n = 0;
  while (find(f, dn_name, layer + n)) n++;
  cfg->layers = n;
  return MOE_OK;
}

namespace {

// Host -> device through two pinned staging buffers: worker threads copy the next chunk out of the file
// mapping (page cache) while the previous one is on its way over PCIe.  A plain hipMemcpy from the
// pageable mapping measures 28 GB/s here; the staged path is used for tensors of at least 64 MiB.
constexpr size_t STAGE_BYTES = (size_t)32 << 20;
constexpr int STAGE_THREADS = 6;

struct Stager {
  void* pin[2] = {nullptr, nullptr};
  hipEvent_t done[2] = {nullptr, nullptr};
  hipStream_t stream = nullptr;
  bool ok = false;
  Stager() {
    ok = hipHostMalloc(&pin[0], STAGE_BYTES, hipHostMallocDefault) == hipSuccess &&
         hipHostMalloc(&pin[1], STAGE_BYTES, hipHostMallocDefault) == hipSuccess &&
         hipEventCreateWithFlags(&done[0], hipEventDisableTiming) == hipSuccess &&
         hipEventCreateWithFlags(&done[1], hipEventDisableTiming) == hipSuccess &&
         hipStreamCreateWithFlags(&stream, hipStreamNonBlocking) == hipSuccess;  // default priority
  }
  ~Stager() {
    if (stream) (void)hipStreamSynchronize(stream);
    for (int i = 0; i < 2; i++) {
      if (done[i]) (void)hipEventDestroy(done[i]);
      if (pin[i]) (void)hipHostFree(pin[i]);
    }
    if (stream) (void)hipStreamDestroy(stream);
  }
  static void fill(uint8_t* dst, const uint8_t* src, size_t n) {
    const size_t per = (n / STAGE_THREADS + 4095) & ~(size_t)4095;
    std::thread th[STAGE_THREADS];
    int nt = 0;
    for (size_t o = 0; o < n; o += per) {
      const size_t m = n - o < per ? n - o : per;
      th[nt++] = std::thread([=] { memcpy(dst + o, src + o, m); });
    }
    for (int i = 0; i < nt; i++) th[i].join();
  }
  int copy(void* dev, const uint8_t* src, size_t n) {
    bool used[2] = {false, false};
    int b = 0;
    for (size_t o = 0; o < n; o += STAGE_BYTES, b ^= 1) {
      const size_t m = n - o < STAGE_BYTES ? n - o : STAGE_BYTES;
      if (used[b]) MOE_HIP(hipEventSynchronize(done[b]));  // the buffer's previous chunk has left
      fill((uint8_t*)pin[b], src + o, m);
      MOE_HIP(hipMemcpyAsync((uint8_t*)dev + o, pin[b], m, hipMemcpyHostToDevice, stream));
      MOE_HIP(hipEventRecord(done[b], stream));
      used[b] = true;
    }
    MOE_HIP(hipStreamSynchronize(stream));
    return MOE_OK;
  }
};

int upload(moe_weights* w, const FTensor& t, hipStream_t st, const uint8_t** dev) {
  void* p = nullptr;
  MOE_HIP(hipMalloc(&p, t.nbytes ? t.nbytes : 1));
  w->dev.push_back(p);
  w->bytes += t.nbytes;
  (void)st;  // set-up work: the copy is complete when this returns
  if (t.nbytes >= ((size_t)64 << 20)) {
    if (!w->stager) w->stager.reset(new (std::nothrow) Stager());
    if (w->stager && w->stager->ok) {
      const int rc = w->stager->copy(p, t.data, t.nbytes);
      if (rc != MOE_OK) return rc;
      *dev = (const uint8_t*)p;
      return MOE_OK;
    }
  }
  // small tensors, or no pinned memory to be had: pageable source, staged by the runtime
  MOE_HIP(hipMemcpy(p, t.data, t.nbytes, hipMemcpyHostToDevice));
  *dev = (const uint8_t*)p;
  return MOE_OK;
}

int hgn_dtype_ok_dense(int dt) { return dt == MOE_DT_BF16 || dt == MOE_DT_F32; }

// f32 -> bf16, round to nearest even, NaN -> 0x7fc0: the rounding the reference applies to the F32 router and
// shared-expert gate tensors of a GGUF file when it builds its bf16 tensors from them (src/gguf_map.h:66-72,145-157)
uint16_t bf16_rne(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// An F32 tensor of the file as bf16 in device memory (host-side rounding, then one copy).
int upload_f32_as_bf16(moe_weights* w, const FTensor& t, const uint8_t** dev) {
  const size_t n = t.nbytes / 4;
  std::vector<uint16_t> h(n);
  for (size_t i = 0; i < n; i++) {
    float v;
    memcpy(&v, t.data + 4 * i, 4);
    h[i] = bf16_rne(v);
  }
  void* p = nullptr;
  MOE_HIP(hipMalloc(&p, n ? n * 2 : 1));
  w->dev.push_back(p);
  w->bytes += n * 2;
  MOE_HIP(hipMemcpy(p, h.data(), n * 2, hipMemcpyHostToDevice));
  *dev = (const uint8_t*)p;
  return MOE_OK;
}

// An f16 vector of the file (an hgn v2 sign-scale plane, dtype 2) as f32 in device memory, as the reference uploads
// its sidecars (src/gpu/parts/30_host_util.inc:824-838)
int upload_f16_as_f32(moe_weights* w, const FTensor& t, uint64_t want_n, const float** dev) {
  if (t.dtype != MOE_DT_F16 || t.nbytes != want_n * 2) return MOE_E_INVALID;
  std::vector<float> h(want_n);
  for (uint64_t i = 0; i < want_n; i++) {
    _Float16 v;
    memcpy(&v, t.data + 2 * i, 2);
    h[i] = (float)v;
  }
  void* p = nullptr;
  MOE_HIP(hipMalloc(&p, want_n ? want_n * 4 : 1));
  w->dev.push_back(p);
  w->bytes += want_n * 4;
  MOE_HIP(hipMemcpy(p, h.data(), want_n * 4, hipMemcpyHostToDevice));
  *dev = (const float*)p;
  return MOE_OK;
}

// An hgn v2 dense tensor (ht with its two f16 planes, or q6g64) -> a bf16 matrix in device memory.  The raw bytes and
// the planes are staged in device memory for the conversion kernel and freed again; only the bf16 matrix stays.
int upload_v2_dense(moe_weights* w, const FTensor& t, const FTensor* su, const FTensor* sv, uint64_t rows, uint64_t cols,
                    hipStream_t st, const uint8_t** dev) {
  uint64_t cells, want;
  if (__builtin_mul_overflow(rows, cols, &cells) || cells > (UINT64_MAX >> 2)) return MOE_E_INVALID;
  if (t.dtype == MOE_DT_HT) {
    if (rows % 128 || cols % 128) return MOE_E_INVALID;
    want = cells / 2;
    if (su->dtype != MOE_DT_F16 || su->nbytes != cols * 2 || sv->dtype != MOE_DT_F16 || sv->nbytes != rows * 2) return MOE_E_INVALID;
  } else {
    if (cols % 64 || __builtin_mul_overflow(rows, ((13 * cols / 16) + 15) & ~15ULL, &want)) return MOE_E_INVALID;
  }
  if (t.nbytes != want) return MOE_E_INVALID;
  void *raw = nullptr, *planes = nullptr, *out = nullptr;
  auto done = [&](int rc) {
    if (raw) (void)hipFree(raw);
    if (planes) (void)hipFree(planes);
    return rc;
  };
  MOE_HIP(hipMalloc(&out, cells * 2));
  w->dev.push_back(out);
  w->bytes += cells * 2;
  if (hipMalloc(&raw, want) != hipSuccess) return done(MOE_E_STATE);
  if (hipMemcpy(raw, t.data, want, hipMemcpyHostToDevice) != hipSuccess) return done(MOE_E_STATE);
  const float *p_su = nullptr, *p_sv = nullptr;
  if (t.dtype == MOE_DT_HT) {
    std::vector<float> h(cols + rows);
    for (uint64_t i = 0; i < cols + rows; i++) {
      _Float16 v;
      memcpy(&v, i < cols ? su->data + 2 * i : sv->data + 2 * (i - cols), 2);
      h[i] = (float)v;
    }
    if (hipMalloc(&planes, h.size() * 4) != hipSuccess) return done(MOE_E_STATE);
    if (hipMemcpy(planes, h.data(), h.size() * 4, hipMemcpyHostToDevice) != hipSuccess) return done(MOE_E_STATE);
    p_su = (const float*)planes;
    p_sv = p_su + cols;
  }
  int rc = moe_v2_dense_to_bf16(t.dtype, (const uint8_t*)raw, p_su, p_sv, rows, cols, (uint16_t*)out, (moe_stream_t)st);
  if (rc == MOE_OK && hipStreamSynchronize(st) != hipSuccess) rc = MOE_E_STATE;
  *dev = (const uint8_t*)out;
  return done(rc);
}

// mtp: the MTP draft layer's MoE, stored as mtp.layers.<i>.mlp.* (src/gpu/parts/40_model.inc:5546-5548,5893)
int load_layer_hgn(moe_ctx* ctx, const moe_file* f, int fl, int cl, moe_weights* w, hipStream_t st, bool mtp) {
  auto findp = [&](const char* leaf) -> const FTensor* {
    char n[160];
    snprintf(n, sizeof n, "%slayers.%d.mlp.%s", mtp ? "mtp." : "", fl, leaf);
    auto it = f->idx.find(n);
    return it == f->idx.end() ? nullptr : &it->second;
  };
  const FTensor* rt = findp("gate.weight");
  const FTensor* gu = findp("experts.gate_up_proj.weight");
  const FTensor* dn = findp("experts.down_proj.weight");
  if (!rt || !gu || !dn) return MOE_E_STATE;
  // routed experts: q4cp, or hgn v2 i4r (both tensors) with its four sign-scale planes
  const bool v2 = gu->dtype == MOE_DT_I4R && dn->dtype == MOE_DT_I4R;
  const auto v2_dense = [](int dt) { return dt == MOE_DT_HT || dt == MOE_DT_Q6G64; };
  if (!(hgn_dtype_ok_dense(rt->dtype) || v2_dense(rt->dtype)) || (!v2 && (gu->dtype != MOE_DT_Q4CP || dn->dtype != MOE_DT_Q4CP)))
    return MOE_E_UNSUPPORTED;
  int rc;
  auto view = [&](const FTensor& t, moe_wview* v, const char* leaf) -> int {
    uint64_t rows, cols;
    if (!matrix_shape(MOE_FILE_HGN, t, rows, cols)) return MOE_E_INVALID;
    if (t.dtype == MOE_DT_HT || t.dtype == MOE_DT_Q6G64) {
      // an hgn v2 dense tensor: converted here, once, to the bf16 matrix the reference's prefill GEMM reads
      // (v2_deq_bf16, src/gpu/parts/30_host_util.inc:1019-1031); planes: <tensor without ".weight">.suh / .svh
      // (30_host_util.inc:840-858)
      const FTensor *su = nullptr, *sv = nullptr;
      if (t.dtype == MOE_DT_HT) {
        std::string base(leaf);
        const std::string sfx = ".weight";
        if (base.size() > sfx.size() && base.compare(base.size() - sfx.size(), sfx.size(), sfx) == 0)
          base.resize(base.size() - sfx.size());
        su = findp((base + ".suh").c_str());
        sv = findp((base + ".svh").c_str());
        if (!su || !sv) return MOE_E_STATE;
      }
      v->dtype = MOE_DT_BF16;
      v->rows = rows;
      v->cols = cols;
      v->scale_stride = 0;
      return upload_v2_dense(w, t, su, sv, rows, cols, st, &v->data);
    }
    v->dtype = t.dtype;
    v->rows = rows;
    v->cols = cols;
    v->scale_stride = t.dtype == MOE_DT_Q4CP ? (((cols / 32 * 2) + 15) & ~15ULL) : 0;
    // the record's byte count must be what the kernels will read for these dims (src/hgn.h:225-233)
    uint64_t want, cells;
    if (__builtin_mul_overflow(rows, cols, &cells)) return MOE_E_INVALID;
    if (t.dtype == MOE_DT_Q4CP) {
      uint64_t sc;
      if (cols % 32 || __builtin_mul_overflow(rows, (uint64_t)v->scale_stride, &sc) ||
          __builtin_add_overflow(64 + cells / 2, sc, &want))
        return MOE_E_INVALID;
    } else if (t.dtype == MOE_DT_I4R) {  // codes, then one fp16 scale per 128 columns, rows unpadded
      if (cols % 128 || __builtin_add_overflow(cells / 2, cells / 128 * 2, &want)) return MOE_E_INVALID;
    } else if (t.dtype == MOE_DT_Q8G32) {  // planar: rows*cols int8 codes, then rows*cols/32 fp16 scales (src/hgn.h:176-183)
      if (cols % 32 || __builtin_add_overflow(cells, cells / 32 * 2, &want)) return MOE_E_INVALID;
    } else if (t.dtype == MOE_DT_Q8G64) {  // per row: cols codes + cols/64 x (fp16 scale, fp16 min) (src/hgn.h:189-196)
      uint64_t stride;
      if (cols % 64 || __builtin_add_overflow(cols, cols / 64 * 4, &stride) || __builtin_mul_overflow(rows, stride, &want))
        return MOE_E_INVALID;
    } else if (__builtin_mul_overflow(cells, (uint64_t)(t.dtype == MOE_DT_F32 ? 4 : 2), &want)) {
      return MOE_E_INVALID;
    }
    if (t.nbytes != want) return MOE_E_INVALID;
    return upload(w, t, st, &v->data);
  };
  moe_wview vr{}, vgu{}, vdn{};
  if ((rc = view(*rt, &vr, "gate.weight")) || (rc = view(*gu, &vgu, "")) || (rc = view(*dn, &vdn, ""))) return rc;
  if ((rc = moe_set_router(ctx, cl, &vr, nullptr))) return rc;
  if (v2) {
    // the planes' names (src/gpu/parts/30_host_util.inc:840-852): <tensor>.suh / <tensor>.svh without the ".weight";
    // the input plane of gate_up_proj is shared by the layer's experts as "experts.su"
    const FTensor* su = findp("experts.gate_up_proj.suh");
    if (!su) su = findp("experts.su");
    const FTensor* svg = findp("experts.gate_up_proj.svh");
    const FTensor* sud = findp("experts.down_proj.suh");
    const FTensor* svd = findp("experts.down_proj.svh");
    if (!su || !svg || !sud || !svd) return MOE_E_STATE;
    const uint64_t d = vgu.cols, mid = vdn.cols;
    const float *p_su, *p_svg, *p_sud, *p_svd;
    if ((rc = upload_f16_as_f32(w, *su, d, &p_su)) || (rc = upload_f16_as_f32(w, *svg, 2 * mid, &p_svg)) ||
        (rc = upload_f16_as_f32(w, *sud, mid, &p_sud)) || (rc = upload_f16_as_f32(w, *svd, d, &p_svd)))
      return rc;
    if ((rc = moe_set_experts_i4r(ctx, cl, &vgu, &vdn, p_su, p_svg, p_sud, p_svd))) return rc;
  } else if ((rc = moe_set_experts_q4cp(ctx, cl, &vgu, &vdn))) {
    return rc;
  }
  const FTensor* sg = findp("shared_expert.gate_proj.weight");
  if (sg) {
    const FTensor* su = findp("shared_expert.up_proj.weight");
    const FTensor* sd = findp("shared_expert.down_proj.weight");
    const FTensor* sx = findp("shared_expert_gate.weight");
    if (!su || !sd || !sx) return MOE_E_STATE;
    // q4cp, or one of the dense dtypes of the reference's generic matvec (bf16, f32, the overlay files' q8g64);
    // moe_set_shared checks that the three agree
    // (an hgn v2 file's ht / q6g64 tensors become bf16 on their way in)
    auto sh_ok = [&](int dt) {
      return dt == MOE_DT_Q4CP || dt == MOE_DT_BF16 || dt == MOE_DT_F32 || dt == MOE_DT_Q8G64 || dt == MOE_DT_Q8G32 || v2_dense(dt);
    };
    if (!sh_ok(sg->dtype) || !sh_ok(su->dtype) || !sh_ok(sd->dtype) || !(hgn_dtype_ok_dense(sx->dtype) || sx->dtype == MOE_DT_Q6G64))
      return MOE_E_UNSUPPORTED;
    // one storage for the three matrices; ht and q6g64 both arrive as bf16 and may be mixed
    const bool all_v2 = v2_dense(sg->dtype) && v2_dense(su->dtype) && v2_dense(sd->dtype);
    if (!all_v2 && (v2_dense(sg->dtype) || v2_dense(su->dtype) || v2_dense(sd->dtype))) return MOE_E_UNSUPPORTED;
    moe_wview a{}, b{}, c2{}, d2{};
    if ((rc = view(*sg, &a, "shared_expert.gate_proj.weight")) || (rc = view(*su, &b, "shared_expert.up_proj.weight")) ||
        (rc = view(*sd, &c2, "shared_expert.down_proj.weight")) || (rc = view(*sx, &d2, "shared_expert_gate.weight")))
      return rc;
    if ((rc = moe_set_shared(ctx, cl, &a, &b, &c2, &d2, 0))) return rc;
  }
  return MOE_OK;
}

int load_layer_gguf(moe_ctx* ctx, const moe_file* f, int fl, int cl, moe_weights* w, hipStream_t st) {
  const FTensor* rt = find(f, "blk.%d.ffn_gate_inp.weight", fl);
  const FTensor* g_ = find(f, "blk.%d.ffn_gate_exps.weight", fl);
  const FTensor* u = find(f, "blk.%d.ffn_up_exps.weight", fl);
  const FTensor* dn = find(f, "blk.%d.ffn_down_exps.weight", fl);
  if (!rt || !g_ || !u || !dn) return MOE_E_STATE;
  if (rt->dtype != 0 && rt->dtype != 30) return MOE_E_UNSUPPORTED;  // F32 / BF16 router
  int rc;
  // raw GGUF blocks are registered by pointer only: the shapes the kernels will read are the
  // context's, so the file's must be exactly those
  moe_config g{};
  if ((rc = moe_get_config(ctx, &g))) return rc;
  auto is = [](const FTensor& t, uint64_t a, uint64_t b, uint64_t c) {
    return t.dims[0] == a && t.dims[1] == b && t.dims[2] == c && t.dims[3] == 1;
  };
  const uint64_t D = (uint64_t)g.d, M = (uint64_t)g.mid, NE = (uint64_t)g.experts;
  if (!is(*rt, D, NE, 1) || !is(*g_, D, M, NE) || !is(*u, D, M, NE) || !is(*dn, M, D, NE)) return MOE_E_INVALID;
  // The reference turns the F32 ffn_gate_inp / ffn_gate_inp_shexp tensors into bf16 when it maps a GGUF file
  // (src/gguf_map.h:9,210-211): its router sees the rounded values, so this loader rounds the same way
  // unless the file object was told to keep F32 (MOE_FILE_OPT_GGUF_F32_ROUTER).
  moe_wview vr{};
  const bool round_rt = rt->dtype == 0 && !f->gguf_keep_f32;
  vr.dtype = (rt->dtype == 0 && !round_rt) ? MOE_DT_F32 : MOE_DT_BF16;
  vr.cols = rt->dims[0];
  vr.rows = rt->dims[1];
  if ((rc = round_rt ? upload_f32_as_bf16(w, *rt, &vr.data) : upload(w, *rt, st, &vr.data))) return rc;
  if ((rc = moe_set_router(ctx, cl, &vr, nullptr))) return rc;
  moe_gg_experts gg{};
  gg.tgu = g_->dtype;
  gg.tdn = dn->dtype;
  if (u->dtype != g_->dtype) return MOE_E_UNSUPPORTED;
  if ((rc = upload(w, *g_, st, &gg.gate)) || (rc = upload(w, *u, st, &gg.up)) || (rc = upload(w, *dn, st, &gg.down))) return rc;
  if ((rc = moe_set_experts_gguf(ctx, cl, &gg))) return rc;  // MOE_E_UNSUPPORTED for types outside Q4_K / Q5_K / Q5_1 / Q8_0
  const FTensor* sg = find(f, "blk.%d.ffn_gate_shexp.weight", fl);
  if (sg) {
    const FTensor* su = find(f, "blk.%d.ffn_up_shexp.weight", fl);
    const FTensor* sd = find(f, "blk.%d.ffn_down_shexp.weight", fl);
    const FTensor* sx = find(f, "blk.%d.ffn_gate_inp_shexp.weight", fl);
    if (!su || !sd || !sx) return MOE_E_STATE;
    // one ggml type for the three shared tensors (moe_set_shared checks that it is a supported one)
    if (su->dtype != sg->dtype || sd->dtype != sg->dtype || (sx->dtype != 0 && sx->dtype != 30))
      return MOE_E_UNSUPPORTED;
    if (!is(*sg, D, M, 1) || !is(*su, D, M, 1) || !is(*sd, M, D, 1) || !is(*sx, D, 1, 1)) return MOE_E_INVALID;
    moe_wview a{}, b{}, c2{}, d2{};
    auto raw = [&](const FTensor& t, moe_wview* v) -> int {
      v->dtype = 0;
      v->cols = t.dims[0];
      v->rows = t.dims[1];
      return upload(w, t, st, &v->data);
    };
    if ((rc = raw(*sg, &a)) || (rc = raw(*su, &b)) || (rc = raw(*sd, &c2))) return rc;
    const bool round_sx = sx->dtype == 0 && !f->gguf_keep_f32;
    d2.cols = sx->dims[0];
    if ((rc = round_sx ? upload_f32_as_bf16(w, *sx, &d2.data) : upload(w, *sx, st, &d2.data))) return rc;
    d2.dtype = (sx->dtype == 0 && !round_sx) ? MOE_DT_F32 : MOE_DT_BF16;
    d2.rows = 1;
    if ((rc = moe_set_shared(ctx, cl, &a, &b, &c2, &d2, sg->dtype))) return rc;
  }
  return MOE_OK;
}

}  // namespace

MOE_API int moe_file_set_option(moe_file* f, int option, int value) {
  if (!f) return MOE_E_INVALID;
  switch (option) {
    case MOE_FILE_OPT_GGUF_F32_ROUTER: f->gguf_keep_f32 = value != 0; return MOE_OK;
    default: return MOE_E_INVALID;
  }
}

MOE_API int moe_weights_free(moe_weights* w) {
  if (!w) return MOE_OK;
  int rc = MOE_OK;
  for (void* p : w->dev) {
    const hipError_t e = hipFree(p);
    if (e != hipSuccess && rc == MOE_OK) rc = (int)e;
  }
  delete w;
  return rc;
}

MOE_API uint64_t moe_weights_bytes(const moe_weights* w) { return w ? w->bytes : 0; }

static int load_layers(moe_ctx* ctx, const moe_file* f, int file_layer0, int ctx_layer0, int n_layers,
                       moe_weights** out, moe_stream_t st, bool mtp) {
  if (!ctx || !f || !out || file_layer0 < 0 || ctx_layer0 < 0 || n_layers < 1) return MOE_E_INVALID;
  moe_weights* w = new (std::nothrow) moe_weights();
  if (!w) return MOE_E_STATE;
  for (int i = 0; i < n_layers; i++) {
    const int rc = f->format == MOE_FILE_HGN ? load_layer_hgn(ctx, f, file_layer0 + i, ctx_layer0 + i, w, moe_s(st), mtp)
                                             : load_layer_gguf(ctx, f, file_layer0 + i, ctx_layer0 + i, w, moe_s(st));
    if (rc != MOE_OK) {
      for (int j = 0; j <= i; j++) (void)moe_clear_layer(ctx, ctx_layer0 + j);  // no layer keeps a freed pointer
      moe_weights_free(w);
      return rc;
    }
  }
  w->stager.reset();  // the staging buffers are not needed once the layers are resident
  *out = w;
  return MOE_OK;
}

MOE_API int moe_load_layers(moe_ctx* ctx, const moe_file* f, int file_layer0, int ctx_layer0, int n_layers,
                            moe_weights** out, moe_stream_t st) {
  return load_layers(ctx, f, file_layer0, ctx_layer0, n_layers, out, st, false);
}

MOE_API int moe_load_mtp_layers(moe_ctx* ctx, const moe_file* f, int mtp_layer0, int ctx_layer0, int n_layers,
                                moe_weights** out, moe_stream_t st) {
  return load_layers(ctx, f, mtp_layer0, ctx_layer0, n_layers, out, st, true);
}
