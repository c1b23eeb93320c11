#include "weights.h"

#include <dirent.h>
#include <errno.h>
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <mutex>

#include "kernels.h"

namespace tq {

uint16_t float_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7F800000u) == 0x7F800000u && (u & 0x7FFFFFu)) return (uint16_t)((u >> 16) | 0x40);       // NaN stays NaN
    u += 0x7FFFu + ((u >> 16) & 1u);             // round to nearest even
    return (uint16_t)(u >> 16);
}

float bf16_to_float(uint16_t b) {
    const uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static float f16_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu, u;
    if (exp == 0) {
        if (man == 0) u = sign;
        else {
            int shift = 0;
            while (!(man & 0x400u)) { man <<= 1; ++shift; }
            man &= 0x3FFu;
            u = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (man << 13);
        }
    } else if (exp == 31) u = sign | 0x7F800000u | (man << 13);
    else u = sign | ((exp + 127 - 15) << 23) | (man << 13);
    float f;
    memcpy(&f, &u, 4);
    return f;
}

// ---- safetensors -----------------------------------------------------------------------------
static const char* const KNOWN_DTYPES[] = {"F32", "BF16", "F16", "F64", "I32", "I64", "I16", "I8", "U8", "BOOL"};

static size_t stored_size(const std::string& dt) {
    if (dt == "F64" || dt == "I64") return 8;
    if (dt == "F32" || dt == "I32") return 4;
    if (dt == "BF16" || dt == "F16" || dt == "I16") return 2;
    return 1;
}

SafetensorsFile::SafetensorsFile(const std::string& path) {
    const int fd = open(path.c_str(), O_RDONLY);
    if (fd < 0) raise(TQE_ERR_WEIGHT_FILE, "Cannot read %s: %s", path.c_str(), strerror(errno));
    struct stat st;
    if (fstat(fd, &st) != 0) { close(fd); raise(TQE_ERR_WEIGHT_FILE, "Cannot read %s: %s", path.c_str(), strerror(errno)); }
    size_ = (size_t)st.st_size;
    if (size_ < 8) { close(fd); raise(TQE_ERR_WEIGHT_FILE, "%s: too short to be a safetensors file", path.c_str()); }
    map_ = mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (map_ == MAP_FAILED) { map_ = nullptr; raise(TQE_ERR_WEIGHT_FILE, "Cannot map %s: %s", path.c_str(), strerror(errno)); }
    const uint8_t* base = (const uint8_t*)map_;
    uint64_t n = 0;
    for (int i = 7; i >= 0; --i) n = (n << 8) | base[i];
    if (n > size_ - 8) raise(TQE_ERR_WEIGHT_FILE, "%s: header length %llu exceeds the file", path.c_str(), (unsigned long long)n);
    Json header;
    try {
        header = Json::parse((const char*)base + 8, (size_t)n);
    } catch (const JsonError& e) {
        raise(TQE_ERR_WEIGHT_FILE, "%s: invalid header: %s", path.c_str(), e.what());
    }
    if (!header.is_object()) raise(TQE_ERR_WEIGHT_FILE, "%s: invalid header: not an object", path.c_str());
    const size_t data_start = 8 + (size_t)n, data_size = size_ - data_start;
    for (const Json::Member& m : header.members()) {
        if (m.first == "__metadata__") continue;
        const Json& info = m.second;
        StoredTensor t;
        t.name = m.first;
        t.dtype = info["dtype"].is_string() ? info["dtype"].as_string() : "";
        bool known = false;
        for (const char* k : KNOWN_DTYPES) known = known || t.dtype == k;
        if (!known) raise(TQE_ERR_WEIGHT_FILE, "%s: tensor %s has unsupported dtype %s", path.c_str(), t.name.c_str(), t.dtype.c_str());
        if (!info["shape"].is_array() || !info["data_offsets"].is_array() || info["data_offsets"].items().size() != 2)
            raise(TQE_ERR_WEIGHT_FILE, "%s: tensor %s has no shape or offsets", path.c_str(), t.name.c_str());
        for (const Json& s : info["shape"].items()) t.shape.push_back(s.as_int());
        const long long begin = info["data_offsets"].items()[0].as_int(), end = info["data_offsets"].items()[1].as_int();
        if (!(0 <= begin && begin <= end && (unsigned long long)end <= data_size))
            raise(TQE_ERR_WEIGHT_FILE, "%s: tensor %s lies outside the file", path.c_str(), t.name.c_str());
        t.data = base + data_start + begin;
        t.bytes = (size_t)(end - begin);
        if ((size_t)t.numel() * stored_size(t.dtype) != t.bytes)
            raise(TQE_ERR_WEIGHT_FILE, "%s: tensor %s holds %zu bytes, its shape asks for %zu", path.c_str(), t.name.c_str(), t.bytes,
                  (size_t)t.numel() * stored_size(t.dtype));
        tensors.push_back(std::move(t));
    }
}

SafetensorsFile::~SafetensorsFile() {
    if (map_) munmap(map_, size_);
}

std::unique_ptr<Folder> open_folder(const std::string& model_dir) {
    DIR* d = opendir(model_dir.c_str());
    if (!d) raise(TQE_ERR_WEIGHT_FILE, "Cannot read model dir: %s: %s", model_dir.c_str(), strerror(errno));
    std::vector<std::string> files;
    while (struct dirent* e = readdir(d)) {
        const std::string name = e->d_name;
        const std::string ext = ".safetensors";
        if (name.size() > ext.size() && name.compare(name.size() - ext.size(), ext.size(), ext) == 0) files.push_back(name);
    }
    closedir(d);
    if (files.empty()) raise(TQE_ERR_WEIGHT_FILE, "No .safetensors files found in %s", model_dir.c_str());
    std::sort(files.begin(), files.end());
    std::unique_ptr<Folder> folder(new Folder());
    for (const std::string& f : files) {
        folder->files.emplace_back(new SafetensorsFile(model_dir + "/" + f));
        for (const StoredTensor& t : folder->files.back()->tensors) folder->tensors[t.name] = t;
    }
    return folder;
}

void write_safetensors(const std::string& path, const std::vector<TensorToWrite>& tensors, const Json& metadata) {
    Json header = Json::object();
    if (metadata.is_object()) header.append("__metadata__", metadata);
    size_t offset = 0;
    for (const TensorToWrite& t : tensors) {
        Json info = Json::object();
        info.set("dtype", t.dtype);
        Json shape = Json::array();
        for (int64_t s : t.shape) shape.push(Json((long long)s));
        info.set("shape", shape);
        Json off = Json::array();
        off.push(Json((long long)offset));
        off.push(Json((long long)(offset + t.bytes)));
        info.set("data_offsets", off);
        header.append(t.name, info);
        offset += t.bytes;
    }
    std::string blob = header.dump();
    while (blob.size() % 8) blob.push_back(' ');
    const std::string tmp = path + format(".tmp%d", (int)getpid());
    FILE* f = fopen(tmp.c_str(), "wb");
    if (!f) raise(TQE_ERR_WEIGHT_FILE, "Cannot write %s: %s", tmp.c_str(), strerror(errno));
    uint8_t len[8];
    uint64_t n = blob.size();
    for (int i = 0; i < 8; ++i) { len[i] = (uint8_t)(n & 0xFF); n >>= 8; }
    bool ok = fwrite(len, 1, 8, f) == 8 && fwrite(blob.data(), 1, blob.size(), f) == blob.size();
    for (const TensorToWrite& t : tensors) {
        if (!ok) break;
        const long before = ftell(f);
        t.write(f);
        ok = !ferror(f) && (size_t)(ftell(f) - before) == t.bytes;
    }
    ok = fclose(f) == 0 && ok;
    if (!ok) { unlink(tmp.c_str()); raise(TQE_ERR_WEIGHT_FILE, "Cannot write %s", path.c_str()); }
    if (rename(tmp.c_str(), path.c_str()) != 0) raise(TQE_ERR_WEIGHT_FILE, "Cannot write %s: %s", path.c_str(), strerror(errno));
}

// ---- loading -----------------------------------------------------------------------------------
int target_dtype(const std::string& stored, const std::string& kind, int run_dtype) {
    if (kind == "int32") return I32;
    if (run_dtype == F32) return F32;
    if (stored == "F32" || stored == "F64") return F32;
    return run_dtype;
}

static std::string shape_text(const std::vector<int64_t>& shape) {
    std::string s = "[";
    for (size_t i = 0; i < shape.size(); ++i) s += format(i ? ", %lld" : "%lld", (long long)shape[i]);
    return s + "]";
}

void check_weights(const std::map<std::string, StoredTensor>& stored, const TensorSpecs& wanted, bool strict, std::string* warning) {
    std::vector<std::string> missing, unexpected, lines;
    Json wrong_shape = Json::array(), wrong_kind = Json::array();
    std::map<std::string, const TensorSpec*> want;
    for (const auto& w : wanted) {
        want[w.first] = &w.second;
        if (!stored.count(w.first)) missing.push_back(w.first);
    }
    for (const auto& s : stored)
        if (!want.count(s.first)) unexpected.push_back(s.first);
    if (!unexpected.empty() && !strict) {
        if (warning) {
            *warning = format("the folder holds %zu tensors the model does not use: ", unexpected.size());
            for (size_t i = 0; i < unexpected.size(); ++i) *warning += (i ? ", " : "") + unexpected[i];
        }
        unexpected.clear();
    }
    lines.push_back("the weights do not fit the model:");
    for (const std::string& n : missing) lines.push_back("  Missing tensor: " + n);
    for (const std::string& n : unexpected) lines.push_back("  Unexpected tensor: " + n);
    std::vector<std::string> shape_lines, kind_lines;
    for (const auto& w : wanted) {
        auto it = stored.find(w.first);
        if (it == stored.end()) continue;
        const StoredTensor& st = it->second;
        if (st.shape != w.second.shape) {
            shape_lines.push_back("  Wrong shape: " + w.first + " is " + shape_text(st.shape) + ", expected " + shape_text(w.second.shape));
            Json e = Json::array();
            e.push(w.first);
            Json got = Json::array(), exp = Json::array();
            for (int64_t v : st.shape) got.push(Json((long long)v));
            for (int64_t v : w.second.shape) exp.push(Json((long long)v));
            e.push(got);
            e.push(exp);
            wrong_shape.push(e);
        }
        if ((w.second.dtype == "float") != st.is_float()) {
            const char* exp = w.second.dtype == "float" ? "a floating type" : "an integer type";
            kind_lines.push_back("  Wrong dtype: " + w.first + " is " + st.dtype + ", expected " + exp);
            Json e = Json::array();
            e.push(w.first);
            e.push(st.dtype);
            e.push(exp);
            wrong_kind.push(e);
        }
    }
    if (missing.empty() && unexpected.empty() && shape_lines.empty() && kind_lines.empty()) return;
    lines.insert(lines.end(), shape_lines.begin(), shape_lines.end());
    lines.insert(lines.end(), kind_lines.begin(), kind_lines.end());
    std::string msg;
    for (size_t i = 0; i < lines.size(); ++i) msg += (i ? "\n" : "") + lines[i];
    Json detail = Json::object();
    Json jm = Json::array(), ju = Json::array();
    for (const std::string& n : missing) jm.push(n);
    for (const std::string& n : unexpected) ju.push(n);
    detail.set("missing", jm);
    detail.set("unexpected", ju);
    detail.set("wrong_shape", wrong_shape);
    detail.set("wrong_kind", wrong_kind);
    throw Error(TQE_ERR_WEIGHTS, msg, detail.dump());
}

// the stored values as `dtype` in host memory (out holds numel values of that type)
static void convert_on_host(const StoredTensor& st, int dtype, void* out) {
    const int64_t n = st.numel();
    const uint8_t* src = st.data;
    auto as_float = [&](int64_t i) -> float {
        if (st.dtype == "F32") { float f; memcpy(&f, src + 4 * i, 4); return f; }
        if (st.dtype == "BF16") { uint16_t b; memcpy(&b, src + 2 * i, 2); return bf16_to_float(b); }
        if (st.dtype == "F16") { uint16_t b; memcpy(&b, src + 2 * i, 2); return f16_to_float(b); }
        if (st.dtype == "F64") { double d; memcpy(&d, src + 8 * i, 8); return (float)d; }
        return 0.f;
    };
    auto as_int = [&](int64_t i) -> long long {
        if (st.dtype == "I64") { int64_t v; memcpy(&v, src + 8 * i, 8); return v; }
        if (st.dtype == "I32") { int32_t v; memcpy(&v, src + 4 * i, 4); return v; }
        if (st.dtype == "I16") { int16_t v; memcpy(&v, src + 2 * i, 2); return v; }
        if (st.dtype == "I8") return (int8_t)src[i];
        return src[i];
    };
    if (dtype == F32) {
        float* o = (float*)out;
        for (int64_t i = 0; i < n; ++i) o[i] = as_float(i);
    } else if (dtype == BF16) {
        uint16_t* o = (uint16_t*)out;
        for (int64_t i = 0; i < n; ++i) o[i] = float_to_bf16(as_float(i));
    } else {
        int32_t* o = (int32_t*)out;
        for (int64_t i = 0; i < n; ++i) o[i] = (int32_t)as_int(i);
    }
}

OwnedPtr upload_tensor(const StoredTensor& st, int dtype, hipStream_t stream) {
    OwnedPtr o = make_owned(dtype, st.shape);
    const bool same = (dtype == F32 && st.dtype == "F32") || (dtype == BF16 && st.dtype == "BF16") || (dtype == I32 && st.dtype == "I32");
    const size_t bytes = o->t.bytes();
    if (bytes == 0) return o;
    if (same) {
        copy_to_device(o->t.data, st.data, bytes, stream);
        stream_synchronize(stream);
        return o;
    }
    // in pieces, so that a large tensor does not need its size again in host memory
    const int64_t n = st.numel(), piece = (int64_t)1 << 22;
    std::vector<uint8_t> host((size_t)std::min(n, piece) * dtype_size(dtype));
    const size_t in_size = stored_size(st.dtype);
    for (int64_t at = 0; at < n; at += piece) {
        StoredTensor part = st;
        part.shape = {std::min(piece, n - at)};
        part.data = st.data + (size_t)at * in_size;
        convert_on_host(part, dtype, host.data());
        copy_to_device((char*)o->t.data + (size_t)at * dtype_size(dtype), host.data(), (size_t)part.shape[0] * dtype_size(dtype), stream);
        stream_synchronize(stream);
    }
    return o;
}

void load_folder(Model& model, const std::string& model_dir, bool strict, std::string* warning, hipStream_t stream) {
    std::unique_ptr<Folder> folder = open_folder(model_dir);
    const TensorSpecs wanted = model.tensor_specs();
    check_weights(folder->tensors, wanted, strict, warning);
    Loaded loaded;
    for (const auto& w : wanted) {
        const StoredTensor& st = folder->tensors.at(w.first);
        loaded[w.first] = upload_tensor(st, target_dtype(st.dtype, w.second.dtype, model.dtype), stream);
    }
    model.load(loaded, stream);
}

// ---- SHA-256 (for a tensor's key) ----------------------------------------------------------------
namespace {
struct Sha256 {
    uint32_t h[8] = {0x6a09e667u, 0xbb67ae85u, 0x3c6ef372u, 0xa54ff53au, 0x510e527fu, 0x9b05688cu, 0x1f83d9abu, 0x5be0cd19u};
    static uint32_t rotr(uint32_t x, int n) { return (x >> n) | (x << (32 - n)); }
    void block(const uint8_t* p) {
        static const uint32_t k[64] = {
            0x428a2f98u, 0x71374491u, 0xb5c0fbcfu, 0xe9b5dba5u, 0x3956c25bu, 0x59f111f1u, 0x923f82a4u, 0xab1c5ed5u, 0xd807aa98u, 0x12835b01u, 0x243185beu,
            0x550c7dc3u, 0x72be5d74u, 0x80deb1feu, 0x9bdc06a7u, 0xc19bf174u, 0xe49b69c1u, 0xefbe4786u, 0x0fc19dc6u, 0x240ca1ccu, 0x2de92c6fu, 0x4a7484aau,
            0x5cb0a9dcu, 0x76f988dau, 0x983e5152u, 0xa831c66du, 0xb00327c8u, 0xbf597fc7u, 0xc6e00bf3u, 0xd5a79147u, 0x06ca6351u, 0x14292967u, 0x27b70a85u,
            0x2e1b2138u, 0x4d2c6dfcu, 0x53380d13u, 0x650a7354u, 0x766a0abbu, 0x81c2c92eu, 0x92722c85u, 0xa2bfe8a1u, 0xa81a664bu, 0xc24b8b70u, 0xc76c51a3u,
            0xd192e819u, 0xd6990624u, 0xf40e3585u, 0x106aa070u, 0x19a4c116u, 0x1e376c08u, 0x2748774cu, 0x34b0bcb5u, 0x391c0cb3u, 0x4ed8aa4au, 0x5b9cca4fu,
            0x682e6ff3u, 0x748f82eeu, 0x78a5636fu, 0x84c87814u, 0x8cc70208u, 0x90befffau, 0xa4506cebu, 0xbef9a3f7u, 0xc67178f2u};
        uint32_t w[64];
        for (int i = 0; i < 16; ++i) w[i] = ((uint32_t)p[4 * i] << 24) | ((uint32_t)p[4 * i + 1] << 16) | ((uint32_t)p[4 * i + 2] << 8) | p[4 * i + 3];
        for (int i = 16; i < 64; ++i) {
            const uint32_t s0 = rotr(w[i - 15], 7) ^ rotr(w[i - 15], 18) ^ (w[i - 15] >> 3);
            const uint32_t s1 = rotr(w[i - 2], 17) ^ rotr(w[i - 2], 19) ^ (w[i - 2] >> 10);
            w[i] = w[i - 16] + s0 + w[i - 7] + s1;
        }
        uint32_t a = h[0], b = h[1], c = h[2], d = h[3], e = h[4], f = h[5], g = h[6], hh = h[7];
        for (int i = 0; i < 64; ++i) {
            const uint32_t t1 = hh + (rotr(e, 6) ^ rotr(e, 11) ^ rotr(e, 25)) + ((e & f) ^ (~e & g)) + k[i] + w[i];
            const uint32_t t2 = (rotr(a, 2) ^ rotr(a, 13) ^ rotr(a, 22)) + ((a & b) ^ (a & c) ^ (b & c));
            hh = g; g = f; f = e; e = d + t1; d = c; c = b; b = a; a = t1 + t2;
        }
        h[0] += a; h[1] += b; h[2] += c; h[3] += d; h[4] += e; h[5] += f; h[6] += g; h[7] += hh;
    }
    void digest(const std::string& msg, uint8_t out[32]) {
        std::string m = msg;
        const uint64_t bits = (uint64_t)msg.size() * 8;
        m.push_back((char)0x80);
        while (m.size() % 64 != 56) m.push_back('\0');
        for (int i = 7; i >= 0; --i) m.push_back((char)((bits >> (8 * i)) & 0xFF));
        for (size_t at = 0; at < m.size(); at += 64) block((const uint8_t*)m.data() + at);
        for (int i = 0; i < 8; ++i) {
            out[4 * i] = (uint8_t)(h[i] >> 24); out[4 * i + 1] = (uint8_t)(h[i] >> 16); out[4 * i + 2] = (uint8_t)(h[i] >> 8); out[4 * i + 3] = (uint8_t)h[i];
        }
    }
};
}  // namespace

// The 64-bit key of a tensor's stream: the first 8 bytes (little-endian) of SHA-256("<seed>:<name>").
uint64_t tensor_key(uint64_t seed, const std::string& name) {
    uint8_t d[32];
    Sha256().digest(format("%llu:", (unsigned long long)seed) + name, d);
    uint64_t key = 0;
    for (int i = 7; i >= 0; --i) key = (key << 8) | d[i];
    return key;
}

// ---- the standard normal stream on the host -------------------------------------------------------
//     x    = mix(key + (i + 1) * GOLDEN)                      (64-bit, wrapping)
//     u1   = ((x >> 40) + 1) / 2^24                  in (0, 1]
//     ln u1 = e * LN2 + t * Q(t),  u1 = m * 2^e,  m in [sqrt(1/2), sqrt(2)),  t = m - 1
//     r    = sqrt(-2 ln u1)  by three Newton steps for 1/sqrt from an integer first guess
//     low 32 bits: quadrant (2 bits) and 23 bits of angle inside it, taken from the middle of a
//                  cell so that the angle is never 0 or pi/2; odd quadrants mirror the angle
//     z    = +-r * C(angle^2)
// Every float32 multiplication and addition is rounded on its own (this file is compiled without
// contraction), as in csrc/random_init.hip.
static inline float horner(const float* coef, int n, float x) {
    volatile float acc = coef[n - 1];
    for (int k = n - 2; k >= 0; --k) {
        acc = acc * x;
        acc = acc + coef[k];
    }
    return acc;
}

static inline int float_bits(float f) { int i; memcpy(&i, &f, 4); return i; }
static inline float bits_float(int i) { float f; memcpy(&f, &i, 4); return f; }

void standard_normal_host(uint64_t key, int64_t begin, int64_t count, float* out) {
    static const float LOG_Q[11] = {1.0f, -0.5f, 0.33333301544189453f, -0.2500002384185791f, 0.2000257670879364f, -0.16668042540550232f,
                                    0.14212606847286224f, -0.1239922046661377f, 0.11923925578594208f, -0.11727229505777359f, 0.06740232557058334f};
    static const float COS_C[7] = {1.0f, -0.5f, 0.0416666679084301f, -0.0013888884568586946f, 2.4801040126476437e-05f, -2.752467764821631e-07f,
                                   1.990758891068367e-09f};
    for (int64_t j = 0; j < count; ++j) {
        uint64_t x = key + ((uint64_t)(begin + j) + 1ull) * 0x9E3779B97F4A7C15ull;
        x ^= x >> 30; x *= 0xBF58476D1CE4E5B9ull;
        x ^= x >> 27; x *= 0x94D049BB133111EBull;
        x ^= x >> 31;
        const uint32_t hi = (uint32_t)(x >> 32), lo = (uint32_t)x;
        const int n = (int)(hi >> 8) + 1;
        const int bits = float_bits((float)n);
        int e = (bits >> 23) - 151;
        volatile float m = bits_float((bits & 0x7FFFFF) | 0x3F800000);
        if (m > 1.4142135f) { m = m * 0.5f; e += 1; }
        const float t = m - 1.0f;
        const float q = horner(LOG_Q, 11, t);
        volatile float a1 = (float)e * 0.6931471805599453f;
        volatile float a2 = t * q;
        const float ln_u = a1 + a2;
        const float v = ln_u * -2.0f;
        volatile float y = bits_float(0x5F3759DF - (float_bits(v) >> 1));
        const float hv = v * 0.5f;
        for (int k = 0; k < 3; ++k) {
            volatile float yy = y * y;
            volatile float p = hv * yy;
            volatile float s = 1.5f - p;
            y = y * s;
        }
        const float r = v * y;
        const uint32_t quadrant = lo >> 30;
        int f = (int)((lo >> 7) & 0x7FFFFFu);
        if (quadrant & 1u) f = 0x7FFFFF - f;
        volatile float frac = (float)(2 * f + 1) * 5.9604644775390625e-08f;
        volatile float a = frac * 1.5707963267948966f;
        volatile float aa = a * a;
        const float c = horner(COS_C, 7, aa);
        const float z = r * c;
        out[j] = (quadrant == 1u || quadrant == 2u) ? -z : z;
    }
}

// ---- init kinds ------------------------------------------------------------------------------------
namespace {
std::map<std::string, InitFill>& init_kinds() {
    static std::map<std::string, InitFill> m;
    return m;
}
std::mutex g_init_mutex;
}  // namespace

void register_init(const std::string& kind, InitFill fill) {
    std::lock_guard<std::mutex> lock(g_init_mutex);
    init_kinds()[kind] = std::move(fill);
}

static InitFill find_init(const std::string& kind) {
    std::lock_guard<std::mutex> lock(g_init_mutex);
    auto it = init_kinds().find(kind);
    return it == init_kinds().end() ? InitFill() : it->second;
}

// count values of a tensor's elements begin.. in float32 on the host
static void fill_host(const std::string& name, const TensorSpec& spec, uint64_t seed, int64_t begin, int64_t count, float* out) {
    if (spec.init == "zeros") { std::fill(out, out + count, 0.f); return; }
    if (spec.init == "normal" || spec.init == "one_plus_normal") {
        standard_normal_host(tensor_key(seed, name), begin, count, out);
        const float sd = (float)spec.std_dev;
        const bool plus = spec.init == "one_plus_normal";
        for (int64_t i = 0; i < count; ++i) {
            volatile float v = out[i] * sd;
            if (plus) v = 1.0f + v;
            out[i] = v;
        }
        return;
    }
    InitFill fill = find_init(spec.init);
    if (!fill) raise(TQE_ERR_ARGUMENT, "unknown init '%s' for tensor %s", spec.init.c_str(), name.c_str());
    fill(name, spec, seed, begin, count, out);
}

static OwnedPtr random_tensor(const std::string& name, const TensorSpec& spec, uint64_t seed, int dtype, hipStream_t stream) {
    if (spec.dtype == "int32") {
        OwnedPtr o = make_owned(I32, spec.shape);
        zero_device(o->t.data, o->t.bytes(), stream);
        return o;
    }
    OwnedPtr o = make_owned(dtype, spec.shape);
    const int64_t n = spec.numel();
    if (n == 0) return o;
    if (spec.init == "zeros") { zero_device(o->t.data, o->t.bytes(), stream); return o; }
    if (!null_device() && (spec.init == "normal" || spec.init == "one_plus_normal")) {
        K::random_normal(o->t.data, dtype, (long long)n, tensor_key(seed, name), (float)spec.std_dev, spec.init == "one_plus_normal" ? 1 : 0, stream);
        return o;
    }
    const int64_t piece = (int64_t)1 << 22;
    std::vector<float> vals((size_t)std::min(n, piece));
    std::vector<uint16_t> half(dtype == BF16 ? vals.size() : 0);
    for (int64_t at = 0; at < n; at += piece) {
        const int64_t cnt = std::min(piece, n - at);
        fill_host(name, spec, seed, at, cnt, vals.data());
        if (dtype == BF16) {
            for (int64_t i = 0; i < cnt; ++i) half[(size_t)i] = float_to_bf16(vals[(size_t)i]);
            copy_to_device((char*)o->t.data + (size_t)at * 2, half.data(), (size_t)cnt * 2, stream);
        } else {
            copy_to_device((char*)o->t.data + (size_t)at * 4, vals.data(), (size_t)cnt * 4, stream);
        }
        stream_synchronize(stream);
    }
    return o;
}

void random_weights(Model& model, uint64_t seed, hipStream_t stream) {
    Loaded loaded;
    for (const auto& w : model.tensor_specs()) loaded[w.first] = random_tensor(w.first, w.second, seed, model.dtype, stream);
    stream_synchronize(stream);
    model.load(loaded, stream);
}

void write_random_folder(const std::string& folder, const std::string& config_text, const TensorSpecs& wanted, uint64_t seed, int store_dtype) {
    if (store_dtype != F32 && store_dtype != BF16) raise(TQE_ERR_ARGUMENT, "random weights are written in float32 or bfloat16");
    if (mkdir(folder.c_str(), 0777) != 0 && errno != EEXIST) {
        // the parents too
        std::string path;
        for (size_t i = 0; i <= folder.size(); ++i)
            if (i == folder.size() || folder[i] == '/') {
                path = folder.substr(0, i);
                if (!path.empty() && mkdir(path.c_str(), 0777) != 0 && errno != EEXIST)
                    raise(TQE_ERR_WEIGHT_FILE, "Cannot make folder %s: %s", path.c_str(), strerror(errno));
            }
    }
    {
        FILE* f = fopen((folder + "/config.json").c_str(), "wb");
        if (!f) raise(TQE_ERR_WEIGHT_FILE, "Cannot write %s/config.json: %s", folder.c_str(), strerror(errno));
        fwrite(config_text.data(), 1, config_text.size(), f);
        fclose(f);
    }
    std::vector<TensorToWrite> list;
    for (const auto& w : wanted) {
        TensorToWrite t;
        t.name = w.first;
        const bool is_int = w.second.dtype == "int32";
        t.dtype = is_int ? "I32" : store_dtype == BF16 ? "BF16" : "F32";
        t.shape = w.second.shape;
        const int64_t n = w.second.numel();
        t.bytes = (size_t)n * (is_int || store_dtype == F32 ? 4 : 2);
        const std::string name = w.first;
        const TensorSpec spec = w.second;
        t.write = [=](FILE* f) {
            const int64_t piece = (int64_t)1 << 20;
            std::vector<float> vals((size_t)std::min<int64_t>(std::max<int64_t>(n, 1), piece));
            std::vector<uint16_t> half(vals.size());
            for (int64_t at = 0; at < n; at += piece) {
                const int64_t cnt = std::min(piece, n - at);
                if (is_int) {
                    std::vector<int32_t> z((size_t)cnt, 0);
                    fwrite(z.data(), 4, (size_t)cnt, f);
                    continue;
                }
                fill_host(name, spec, seed, at, cnt, vals.data());
                if (store_dtype == BF16) {
                    for (int64_t i = 0; i < cnt; ++i) half[(size_t)i] = float_to_bf16(vals[(size_t)i]);
                    fwrite(half.data(), 2, (size_t)cnt, f);
                } else {
                    fwrite(vals.data(), 4, (size_t)cnt, f);
                }
            }
        };
        list.push_back(std::move(t));
    }
    Json meta = Json::object();
    meta.set("format", "pt");
    meta.set("seed", format("%llu", (unsigned long long)seed));
    write_safetensors(folder + "/model.safetensors", list, meta);
}

}  // namespace tq
