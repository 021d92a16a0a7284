// Run-time compilation and the kernel cache.
//
// The reference turns generated CUDA C into a cubin by forking `nvcc`, keyed by
// (compute capability, MD5 of the text), with a table in memory and a
// directory on disk (Compile.hs:543-594, Persistent.hs:77-137,218-228,305-378).
// Here the compiler is hiprtc, in process, and the key is a SHA-256 over
// everything that decides the code object: library version, target ISA,
// compiler version, the options, the embedded device headers and the text.
//
// Disk format of <dir>/<target>/<key>.co:
//     "ACCHIPCO" | u64 payload size | 32-byte SHA-256 of payload | payload
// A file is written under a temporary name and renamed into place, so a crash
// never leaves a half-written entry under its final name; an entry whose size
// or hash does not check out is deleted and compiled afresh.  (The reference's
// index file is rewritten in place and is not crash-safe, Persistent.hs:368-378.)
#include <sys/stat.h>
#include <sys/types.h>
#include <unistd.h>

#include <atomic>
#include <cerrno>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <memory>
#include <unordered_map>

#include "acc_internal.hpp"
#include "sha256.hpp"

namespace acc {
namespace {

struct Cache {
  std::mutex mu;
  std::unordered_map<std::string, std::shared_ptr<std::vector<char>>> ram;
  std::vector<std::shared_ptr<std::vector<char>>> retired;   // keeps pointers handed out alive
  std::string dir;
  bool dir_set = false;
  acc_cache_stats stats = {0, 0, 0, 0};
};

Cache &cache()
{
  static Cache c;
  return c;
}

bool mkdirs(const std::string &path)
{
  std::string cur;
  for (size_t i = 0; i <= path.size(); ++i) {
    if (i == path.size() || path[i] == '/') {
      if (!cur.empty() && cur != "/") {
        if (mkdir(cur.c_str(), 0755) != 0 && errno != EEXIST) return false;
      }
    }
    if (i < path.size()) cur.push_back(path[i]);
  }
  struct stat st;
  return stat(path.c_str(), &st) == 0 && S_ISDIR(st.st_mode);
}

std::string default_dir()
{
  if (const char *e = std::getenv("ACC_HIP_CACHE_DIR")) return e;
  const char *home = std::getenv("HOME");
  if (!home || !*home) return "";
  // same place the reference keeps its cache: ~/.accelerate/<package>-<version>/cache
  return std::string(home) + "/.accelerate/accelerate-hip-" ACC_HIP_VERSION "/cache";
}

const std::string &dir_locked(Cache &c)
{
  if (!c.dir_set) { c.dir = default_dir(); c.dir_set = true; }
  return c.dir;
}

const char kMagic[8] = {'A', 'C', 'C', 'H', 'I', 'P', 'C', 'O'};

bool read_entry(const std::string &path, std::vector<char> *payload)
{
  std::ifstream in(path, std::ios::binary);
  if (!in) return false;
  char magic[8];
  uint64_t size = 0;
  uint8_t want[32], got[32];
  in.read(magic, 8);
  in.read(reinterpret_cast<char *>(&size), 8);
  in.read(reinterpret_cast<char *>(want), 32);
  if (!in || std::memcmp(magic, kMagic, 8) != 0 || size == 0 || size > (1ull << 30)) return false;
  payload->resize(size);
  in.read(payload->data(), static_cast<std::streamsize>(size));
  if (!in || in.gcount() != static_cast<std::streamsize>(size)) return false;
  char extra;
  in.read(&extra, 1);
  if (in.gcount() != 0) return false;   // trailing bytes
  Sha256 h;
  h.update(payload->data(), payload->size());
  h.digest(got);
  return std::memcmp(want, got, 32) == 0;
}

bool write_entry(const std::string &dir, const std::string &path, const std::vector<char> &payload)
{
  if (!mkdirs(dir)) return false;
  // unique per process and per call: two threads may be writing the same entry
  static std::atomic<unsigned long> serial{0};
  const std::string tmp = path + ".tmp." + std::to_string(static_cast<long>(getpid())) + "." + std::to_string(serial.fetch_add(1));
  {
    std::ofstream out(tmp, std::ios::binary | std::ios::trunc);
    if (!out) return false;
    uint64_t size = payload.size();
    uint8_t dg[32];
    Sha256 h;
    h.update(payload.data(), payload.size());
    h.digest(dg);
    out.write(kMagic, 8);
    out.write(reinterpret_cast<const char *>(&size), 8);
    out.write(reinterpret_cast<const char *>(dg), 32);
    out.write(payload.data(), static_cast<std::streamsize>(payload.size()));
    out.flush();
    if (!out) { unlink(tmp.c_str()); return false; }
  }
  if (rename(tmp.c_str(), path.c_str()) != 0) { unlink(tmp.c_str()); return false; }
  return true;
}

int run_hiprtc(const std::string &target, const char *source, const std::vector<std::string> &options,
               std::vector<char> *code)
{
  const std::vector<EmbeddedHeader> &hdrs = embedded_headers();
  std::vector<std::string> texts;
  std::vector<const char *> text_ptrs, names;
  for (const EmbeddedHeader &h : hdrs) texts.emplace_back(h.begin, h.end);
  for (size_t i = 0; i < hdrs.size(); ++i) { text_ptrs.push_back(texts[i].c_str()); names.push_back(hdrs[i].name); }

  hiprtcProgram prog;
  hiprtcResult r = hiprtcCreateProgram(&prog, source, "accelerate_skeleton.hip", static_cast<int>(hdrs.size()),
                                       text_ptrs.data(), names.data());
  if (r != HIPRTC_SUCCESS) return fail(ACC_ERR_COMPILE, "hiprtcCreateProgram: %s", hiprtcGetErrorString(r));

  std::vector<std::string> opts = options;
  opts.push_back("--offload-arch=" + target);
  std::vector<const char *> optp;
  for (const std::string &o : opts) optp.push_back(o.c_str());
  r = hiprtcCompileProgram(prog, static_cast<int>(optp.size()), optp.data());

  size_t log_size = 0;
  std::string log;
  if (hiprtcGetProgramLogSize(prog, &log_size) == HIPRTC_SUCCESS && log_size > 1) {
    log.resize(log_size);
    hiprtcGetProgramLog(prog, &log[0]);
    while (!log.empty() && log.back() == '\0') log.pop_back();
  }
  set_compile_log(log);
  if (r != HIPRTC_SUCCESS) {
    hiprtcDestroyProgram(&prog);
    // nvcc's exit status reaches the waiting thread as an error in the
    // reference (Compile.hs:643-646,665-670); here it is a status plus the log
    return fail(ACC_ERR_COMPILE, "run-time compilation failed (%s); see acc_compile_log()", hiprtcGetErrorString(r));
  }
  size_t size = 0;
  r = hiprtcGetCodeSize(prog, &size);
  if (r == HIPRTC_SUCCESS && size) {
    code->resize(size);
    r = hiprtcGetCode(prog, code->data());
  }
  hiprtcDestroyProgram(&prog);
  if (r != HIPRTC_SUCCESS || size == 0) return fail(ACC_ERR_COMPILE, "hiprtcGetCode: %s", hiprtcGetErrorString(r));
  return ACC_OK;
}

}  // namespace

int compile_in_process(const std::string &target, const char *source, const std::vector<std::string> &options, std::vector<char> *code)
{
  return run_hiprtc(target, source, options, code);
}

}  // namespace acc

using acc::fail;

extern "C" {

int acc_cache_set_dir(const char *dir)
{
  acc::Cache &c = acc::cache();
  std::lock_guard<std::mutex> lock(c.mu);
  c.dir = dir ? dir : "";
  c.dir_set = true;
  return ACC_OK;
}

const char *acc_cache_dir(void)
{
  acc::Cache &c = acc::cache();
  std::lock_guard<std::mutex> lock(c.mu);
  return acc::dir_locked(c).c_str();
}

int acc_cache_get_stats(acc_cache_stats *out)
{
  if (!out) return fail(ACC_ERR_INVALID, "acc_cache_get_stats: NULL argument");
  acc::Cache &c = acc::cache();
  std::lock_guard<std::mutex> lock(c.mu);
  *out = c.stats;
  return ACC_OK;
}

int acc_cache_clear(int also_disk)
{
  acc::Cache &c = acc::cache();
  std::lock_guard<std::mutex> lock(c.mu);
  for (auto &kv : c.ram) {
    if (also_disk) {
      const std::string &dir = acc::dir_locked(c);
      if (!dir.empty()) unlink((dir + "/" + kv.first).c_str());   // key already carries "<target>/<hash>.co"
    }
    c.retired.push_back(kv.second);
  }
  c.ram.clear();
  return ACC_OK;
}

int acc_compile(acc_context ctx, const char *target, const char *source, const char *const *options, int n_options,
                const void **code, size_t *code_size)
{
  if (!source || !code || !code_size || n_options < 0 || (n_options > 0 && !options))
    return fail(ACC_ERR_INVALID, "acc_compile: bad argument");
  std::string tgt;
  if (target && *target) tgt = target;
  else if (ctx) tgt = ctx->arch;
  else return fail(ACC_ERR_INVALID, "acc_compile: no target and no context");
  for (char ch : tgt)
    if (!(isalnum(static_cast<unsigned char>(ch)) || ch == '_' || ch == '-' || ch == '+' || ch == ':'))
      return fail(ACC_ERR_INVALID, "acc_compile: bad target name '%s'", tgt.c_str());

  std::vector<std::string> opts;
  for (int i = 0; i < n_options; ++i) opts.emplace_back(options[i] ? options[i] : "");

  int rtc_major = 0, rtc_minor = 0;
  hiprtcVersion(&rtc_major, &rtc_minor);

  acc::Sha256 h;
  h.field("accelerate-hip " ACC_HIP_VERSION);
  h.field(tgt);
  h.field(std::to_string(rtc_major) + "." + std::to_string(rtc_minor));
  for (const std::string &o : opts) h.field(o);
  h.field("--");
  // (the device headers enter the key through their own digest, worked out once: they are 150 KB, a source is 3)
  static const std::string headers_digest = [] {
    acc::Sha256 hh;
    for (const acc::EmbeddedHeader &eh : acc::embedded_headers()) {
      hh.field(eh.name);
      hh.field(std::string(eh.begin, eh.end));
    }
    return hh.hex();
  }();
  h.field(headers_digest);
  h.field(source);
  const std::string key = tgt + "/" + h.hex() + ".co";

  acc::Cache &c = acc::cache();
  std::string dir;
  {
    std::lock_guard<std::mutex> lock(c.mu);
    auto it = c.ram.find(key);
    if (it != c.ram.end()) {
      ++c.stats.ram_hits;
      *code = it->second->data();
      *code_size = it->second->size();
      acc::set_compile_log("");
      return ACC_OK;
    }
    dir = acc::dir_locked(c);
  }

  auto payload = std::make_shared<std::vector<char>>();
  bool from_disk = false;
  bool disk_error = false;
  const std::string path = dir.empty() ? std::string() : dir + "/" + key;
  if (!path.empty()) {
    struct stat st;
    if (stat(path.c_str(), &st) == 0) {
      if (acc::read_entry(path, payload.get())) from_disk = true;
      else { disk_error = true; unlink(path.c_str()); payload->clear(); }
    }
  }
  if (!from_disk) {
    // the lock is not held while compiling: several threads may compile at
    // once, as the reference's worker pool does (Compile.hs:620-660)
    // (a thread of the worker pool hands the job to its helper process: hiprtc takes one program at a time per process)
    int crc = ACC_OK;
    std::string clog;
    if (acc::compile_out_of_process(tgt, source, opts, payload.get(), &clog, &crc)) {
      acc::set_compile_log(clog);
      if (crc != ACC_OK) return fail(crc, "run-time compilation failed; see acc_compile_log()");
    } else {
      ACC_TRY(acc::run_hiprtc(tgt, source, opts, payload.get()));
    }
    if (!path.empty() && !acc::write_entry(dir + "/" + tgt, path, *payload)) disk_error = true;
  } else {
    acc::set_compile_log("");
  }

  std::lock_guard<std::mutex> lock(c.mu);
  if (disk_error) ++c.stats.disk_errors;
  if (from_disk) ++c.stats.disk_hits; else ++c.stats.compiles;
  auto ins = c.ram.emplace(key, payload);   // a racing thread may have inserted the same key: keep the first
  *code = ins.first->second->data();
  *code_size = ins.first->second->size();
  return ACC_OK;
}

}  // extern "C"
