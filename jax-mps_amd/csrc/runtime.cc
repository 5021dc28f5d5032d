// Device singleton, caching allocator, kernel cache, and the plan executor.
#include "runtime.h"

#include <dlfcn.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <chrono>
#include <functional>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <thread>

namespace mi355 {

namespace {

void check(int rc, const char* what) {
  if (rc != 0) throw RuntimeError(std::string(what) + " failed: " + mi355_last_error());
}

uint64_t fnv1a(const std::string& s, uint64_t seed) {
  uint64_t h = seed;
  for (unsigned char c : s) { h ^= c; h *= 1099511628211ull; }
  return h;
}

std::string libraryDir() {
  Dl_info info;
  if (dladdr((void*)&fnv1a, &info) && info.dli_fname) {
    std::string p = info.dli_fname;
    auto k = p.rfind('/');
    if (k != std::string::npos) return p.substr(0, k);
  }
  return ".";
}

// On-disk cache of code objects keyed by the kernel source.  Populated at build time
// (cross-compilation needs no GPU) and at run time for kernels seen for the first time.
std::string cacheDir() {
  static std::string dir = [] {
    const char* e = getenv("MI355X_KERNEL_CACHE_DIR");
    std::string d = e ? std::string(e) : libraryDir() + "/kcache";
    if (d == "off" || d.empty()) return std::string();
    mkdir(d.c_str(), 0755);
    return d;
  }();
  return dir;
}

std::string cachePath(const std::string& source, const std::string& arch) {
  std::string d = cacheDir();
  if (d.empty()) return "";
  char name[80];
  const std::string target = arch + "|" + mi355_rtc_fingerprint();   // a code object is only valid for the compiler that made it
  snprintf(name, sizeof name, "/%016llx%016llx.hsaco", (unsigned long long)fnv1a(source + target, 14695981039346656037ull),
           (unsigned long long)fnv1a(target + source, 0x9E3779B97F4A7C15ull));
  return d + name;
}

bool readFile(const std::string& path, std::vector<char>& out) {
  std::ifstream f(path, std::ios::binary);
  if (!f) return false;
  f.seekg(0, std::ios::end);
  std::streamsize n = f.tellg();
  if (n <= 0) return false;
  f.seekg(0);
  out.resize((size_t)n);
  f.read(out.data(), n);
  return (bool)f;
}

void writeFileAtomic(const std::string& path, const char* data, size_t n) {
  std::string tmp = path + ".tmp" + std::to_string((long)getpid()) + "_" + std::to_string((unsigned long)(uintptr_t)data);
  {
    std::ofstream f(tmp, std::ios::binary);
    if (!f) return;
    f.write(data, (std::streamsize)n);
    if (!f) { unlink(tmp.c_str()); return; }
  }
  if (rename(tmp.c_str(), path.c_str()) != 0) unlink(tmp.c_str());
}

std::string baseArch(const std::string& arch) {
  auto k = arch.find(':');
  return k == std::string::npos ? arch : arch.substr(0, k);
}

}  // namespace

// Compiles every kernel source that is not cached on disk yet; returns the code objects.
// Needs no GPU, so the build step can run it ahead of time.
std::vector<std::vector<char>> compileKernelSources(const std::vector<const std::string*>& sources, const std::string& arch,
                                                    int* fromDisk, int* compiled) {
  size_t n = sources.size();
  std::vector<std::vector<char>> code(n);
  std::vector<std::string> errors(n);
  std::atomic<size_t> next{0};
  std::atomic<int> nDisk{0}, nComp{0};
  unsigned hw = std::thread::hardware_concurrency();
  unsigned workers = std::max(1u, std::min<unsigned>({hw ? hw : 4u, 16u, (unsigned)n}));
  auto work = [&] {
    while (true) {
      size_t i = next.fetch_add(1);
      if (i >= n) break;
      std::string path = cachePath(*sources[i], arch);
      if (!path.empty() && readFile(path, code[i])) { nDisk++; continue; }
      char* buf = nullptr;
      size_t sz = 0;
      std::vector<char> log(1 << 14);
      int rc = mi355_rtc_compile(sources[i]->c_str(), arch.c_str(), &buf, &sz, log.data(), log.size());
      if (rc != 0) {
        errors[i] = std::string("kernel compilation failed: ") + mi355_last_error();
        if (getenv("MI355X_DUMP_KERNELS")) fprintf(stderr, "---- failing kernel ----\n%s\n", sources[i]->c_str());
        continue;
      }
      code[i].assign(buf, buf + sz);
      free(buf);
      nComp++;
      if (!path.empty()) writeFileAtomic(path, code[i].data(), code[i].size());
    }
  };
  std::vector<std::thread> pool;
  for (unsigned w = 1; w < workers; ++w) pool.emplace_back(work);
  work();
  for (auto& t : pool) t.join();
  for (size_t i = 0; i < n; ++i)
    if (!errors[i].empty()) throw RuntimeError(errors[i] + "\n---- source ----\n" + *sources[i]);
  if (fromDisk) *fromDisk = nDisk;
  if (compiled) *compiled = nComp;
  return code;
}

// ---------------------------------------------------------------- Device
bool Device::available(std::string* why) {
  int n = 0;
  if (mi355_device_count(&n) != 0 || n <= 0) {
    if (why) *why = std::string("no HIP device: ") + mi355_last_error();
    return false;
  }
  return true;
}

Device& Device::get() {
  static Device* d = new Device();   // never destroyed: buffers may outlive static destruction order
  return *d;
}

Device::Device() {
  std::string why;
  if (!available(&why)) throw RuntimeError("MI355X plugin: " + why + " (this plugin has no CPU fallback)");
  char name[256], arch[256];
  check(mi355_device_init(0, name, sizeof name, arch, sizeof arch, &cus_, &totalMem_), "device init");
  // resolve the fixed workspace of mi355x_scatter_rows_noalloc now; a failure is reported by that entry point's first call
  (void)mi355_noalloc_setup();
  name_ = name;
  arch_ = arch;
  if (baseArch(arch_) != "gfx950")
    throw RuntimeError("MI355X plugin: device architecture is " + arch_ + "; the kernels of this library are built for gfx950 only");
  check(mi355_stream_create(&stream_), "stream create");
  check(mi355_host_alloc(&pinned_, 4096), "pinned alloc");
}

void* Device::alloc(size_t bytes) {
  size_t sz = std::max<size_t>(256, (bytes + 255) / 256 * 256);
  std::lock_guard<std::mutex> lk(mu_);
  void* p = nullptr;
  auto it = free_.lower_bound(sz);
  // reuse a cached block if it is not wastefully large; among blocks of that size the one released last (equal keys keep
  // their insertion order): a train step that releases its old state and allocates its new one then sees the same few
  // address sets over and over, whatever else sits in the pool, which is what lets captured graphs be replayed
  if (it != free_.end() && it->first <= sz + sz / 4 + 4096) {
    it = std::prev(free_.upper_bound(it->first));
    p = it->second;
    sz = it->first;
    free_.erase(it);
  } else {
    int rc = mi355_malloc(&p, sz);
    if (rc != 0) {
      // give cached blocks back and retry once
      for (auto& kv : free_) { mi355_free(kv.second); sizes_.erase(kv.second); reserved_ -= (int64_t)kv.first; }
      free_.clear();
      check(mi355_malloc(&p, sz), "device allocation");
    }
    sizes_[p] = sz;
    reserved_ += (int64_t)sz;
  }
  inUse_ += (int64_t)sz;
  peak_ = std::max(peak_, inUse_);
  numAllocs_++;
  largest_ = std::max<int64_t>(largest_, (int64_t)sz);
  return p;
}

void Device::release(void* ptr) {
  if (!ptr) return;
  std::lock_guard<std::mutex> lk(mu_);
  auto it = sizes_.find(ptr);
  if (it == sizes_.end()) return;
  inUse_ -= (int64_t)it->second;
  // Every use of a block is ordered on the main stream: work a plan puts on its second stream is joined into the
  // main stream before execute returns or throws (Executable::runPlan).  So a recycled block is only touched by
  // work that is ordered after everything that used it before.
  free_.emplace(it->second, ptr);
}

void Device::sync() { check(mi355_stream_sync(stream_), "stream synchronize"); }

mi355_function_t Device::findKernel(const std::string& source) {
  std::lock_guard<std::mutex> lk(mu_);
  auto it = kernels_.find(source);
  return it == kernels_.end() ? nullptr : it->second;
}
void Device::storeKernel(const std::string& source, mi355_function_t fn) {
  std::lock_guard<std::mutex> lk(mu_);
  kernels_[source] = fn;
}

DeviceBuffer::~DeviceBuffer() {
  if (ptr) Device::get().release(ptr);
}

// ------------------------------------------------------------- Executable
Executable::Executable(std::unique_ptr<CompiledProgram> prog) : prog_(std::move(prog)) {
  Device& dev = Device::get();
  const char* t = getenv("MI355X_TIMING");
  timingKinds_ = t ? t : "";
  const char* every = getenv("MI355X_TIMING_EVERY");   // time one execute call in N (sampling keeps the events' own cost small)
  timingEvery_ = every ? std::max(1, atoi(every)) : 1;
  const char* repeat = getenv("MI355X_TIMING_REPEAT");   // launches of a timed fused kernel per event pair
  timingRepeat_ = repeat ? std::max(1, atoi(repeat)) : 1;
  const char* rot = getenv("MI355X_TIMING_ROTATE_BYTES");
  rotateBytes_ = rot ? std::max<long long>(0, atoll(rot)) : 0;
  // Whole-plan graphs are opt-in (read when the executable is made): measured on this device a graph of a loop-free
  // plan replays no faster than its launches in stream order (MLP step 44 -> 50 us, embedding 90 -> 97 us, ResNet18
  // 4.79 -> 4.87 ms, DistilBERT unchanged): the cost of a dependent launch is on the device, not in the host's calls.
  const char* pg = getenv("MI355X_PLAN_GRAPHS");
  planGraphsOn_ = pg && atoi(pg) != 0;
  const char* gr = getenv("MI355X_GRAPHS");   // "0" runs loop bodies launch by launch
  useGraphs_ = !(gr && gr[0] == '0');
  loadKernels();
  if (prog_->arenaBytes > 0) arena_ = dev.alloc((size_t)prog_->arenaBytes);
  if (!prog_->constPool.empty()) {
    consts_ = dev.alloc(prog_->constPool.size());
    check(mi355_memcpy_h2d(consts_, prog_->constPool.data(), prog_->constPool.size(), dev.stream()), "constant upload");
    dev.sync();
  }
}

Executable::~Executable() {
  Device& dev = Device::get();
  // the arena may still be in use by queued work
  try { dev.sync(); } catch (...) {}
  if (arena_) dev.release(arena_);
  if (consts_) dev.release(consts_);
  for (auto& sh : shadows_) {
    for (void* p : sh.params) dev.release(p);
    for (void* p : sh.outs) dev.release(p);
    if (sh.arena) dev.release(sh.arena);
  }
  for (auto& g : loopGraphs_) for (auto& e : g.second.entries) if (e.exec) mi355_graph_destroy(e.exec);
  for (auto& g : planGraphs_) if (g.exec) mi355_graph_destroy(g.exec);
  for (auto e : eventPool_) mi355_event_destroy(e);
  for (auto& p : pending_) { mi355_event_destroy(p.a); mi355_event_destroy(p.b); }
  // (work on the second stream was joined into the main stream before each call returned, so it has drained too)
  for (auto e : forkStart_) mi355_event_destroy(e);
  for (auto e : forkDone_) mi355_event_destroy(e);
  if (sideStream_) mi355_stream_destroy(sideStream_);
}

void Executable::loadKernels() {
  Device& dev = Device::get();
  auto t0 = std::chrono::steady_clock::now();
  std::vector<const std::string*> todo;
  std::vector<size_t> idx;
  for (size_t i = 0; i < prog_->kernels.size(); ++i) {
    auto& k = prog_->kernels[i];
    k.function = dev.findKernel(k.source);
    if (!k.function) { todo.push_back(&k.source); idx.push_back(i); }
  }
  int fromDisk = 0, compiled = 0;
  auto code = compileKernelSources(todo, baseArch(dev.arch()), &fromDisk, &compiled);
  for (size_t q = 0; q < idx.size(); ++q) {
    auto& k = prog_->kernels[idx[q]];
    mi355_function_t fn = nullptr;
    check(mi355_module_load(code[q].data(), &fn), "module load");
    k.function = fn;
    dev.storeKernel(k.source, fn);
  }
  compileSeconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
  if (getenv("MI355X_VERBOSE"))
    fprintf(stderr, "[mi355x] %zu fused kernels (%d compiled, %d from disk cache, %zu shared) in %.2f s; %d steps, arena %.1f MiB\n",
            prog_->kernels.size(), compiled, fromDisk, prog_->kernels.size() - idx.size(), compileSeconds, prog_->numSteps,
            prog_->arenaBytes / 1048576.0);
}

void* Executable::resolve(const BufRef& r, const std::vector<DeviceBuffer*>& in, const std::vector<void*>& out) const {
  // inside a loop whose counter the host follows, some addresses move with the iteration
  const int64_t moved = r.ivTable < 0 ? 0 : prog_->ivTables[(size_t)r.ivTable][(size_t)std::min<int64_t>(hostIteration_, (int64_t)prog_->ivTables[(size_t)r.ivTable].size() - 1)];
  switch (r.kind) {
    case BufRef::Param: return (char*)in[r.index]->ptr + r.offset + moved;
    case BufRef::Output: return (char*)out[r.index] + r.offset + moved;
    case BufRef::Temp: return (char*)arena_ + r.offset + moved;
    case BufRef::Const: return (char*)consts_ + r.offset + moved;
    default: return nullptr;
  }
}

void* Executable::resolveIn(const BufRef& r, int set, const std::vector<DeviceBuffer*>& in, const std::vector<void*>& out) const {
  if (set == 0 || shadows_.empty()) return resolve(r, in, out);
  const ShadowSet& sh = shadows_[(size_t)set - 1];
  switch (r.kind) {
    case BufRef::Param: return (char*)sh.params[(size_t)r.index] + r.offset;
    case BufRef::Output: return (char*)sh.outs[(size_t)r.index] + r.offset;
    case BufRef::Temp: return (char*)sh.arena + r.offset;
    default: return resolve(r, in, out);
  }
}

// Copies of the call's arguments (same contents), results and arena, until all sets together hold rotateBytes_.
void Executable::prepareShadows(const std::vector<DeviceBuffer*>& in) {
  if (rotateBytes_ <= 0 || !shadows_.empty()) return;
  Device& dev = Device::get();
  int64_t perSet = prog_->arenaBytes;
  for (auto& t : prog_->paramTypes) perSet += (int64_t)t.bytes();
  for (auto& o : prog_->outputs) perSet += (int64_t)o.type.bytes();
  if (perSet <= 0) return;
  int64_t sets = std::max<int64_t>(3, (rotateBytes_ + perSet - 1) / perSet);
  sets = std::min<int64_t>(sets, 256);
  for (int64_t k = 1; k < sets; ++k) {
    ShadowSet sh;
    for (size_t i = 0; i < in.size(); ++i) {
      size_t bytes = std::max<size_t>(prog_->paramTypes[i].bytes(), 4);
      void* p = dev.alloc(bytes);
      check(mi355_memcpy_d2d(p, in[i]->ptr, prog_->paramTypes[i].bytes(), dev.stream()), "shadow copy");
      sh.params.push_back(p);
    }
    for (auto& o : prog_->outputs) sh.outs.push_back(dev.alloc(std::max<size_t>(o.type.bytes(), 4)));
    if (prog_->arenaBytes > 0) sh.arena = dev.alloc((size_t)prog_->arenaBytes);
    shadows_.push_back(std::move(sh));
  }
}

bool Executable::timed(const std::string& kind) const {
  if (timingKinds_.empty()) return false;
  if (timingKinds_ == "all" || timingKinds_ == "1") return true;
  return ("," + timingKinds_ + ",").find("," + kind + ",") != std::string::npos;
}

mi355_event_t Executable::getEvent() {
  if (!eventPool_.empty()) {
    auto e = eventPool_.back();
    eventPool_.pop_back();
    return e;
  }
  mi355_event_t e;
  check(mi355_event_create(&e, 1), "event create");
  return e;
}

void Executable::resolvePending() {
  if (pending_.empty()) return;
  Device::get().sync();
  for (auto& p : pending_) {
    float ms = 0;
    if (mi355_event_elapsed_ms(p.a, p.b, &ms) == 0) {
      auto& s = stats_[p.kind];
      s.count += (int64_t)p.launches;
      s.ms += ms;
      s.flops += p.flops;
      s.bytes += p.bytes;
    }
    eventPool_.push_back(p.a);
    eventPool_.push_back(p.b);
  }
  pending_.clear();
}

std::map<std::string, KindStat> Executable::timings() {
  std::lock_guard<std::mutex> lk(mu_);
  resolvePending();
  return stats_;
}

static int dtypeCode(DType d) { return abiDtypeCode(d); }

void Executable::runStep(const Step& s, const std::vector<DeviceBuffer*>& in, const std::vector<void*>& out) {
  Device& dev = Device::get();
  mi355_stream_t st = streamOverride_ ? streamOverride_ : dev.stream();
  std::string kind;
  double flops = 0, bytes = 0;
  switch (s.kind) {
    case Step::Kernel: kind = s.label.rfind("reduce", 0) == 0 ? "reduce" : "fusion"; bytes = (double)s.algoBytes; break;
    case Step::Gemm: kind = "gemm"; flops = 2.0 * s.gemm.batch0 * s.gemm.batch1 * s.gemm.M * s.gemm.N * (s.gemm.K + (s.dual ? s.gemm2.K : 0)); break;
    case Step::Attention: kind = "attention"; flops = 4.0 * s.attn.B * s.attn.N * s.attn.T * s.attn.S * s.attn.H; break;
    case Step::GemmGroup:
      kind = "gemm";
      for (auto& part : s.parts) flops += 2.0 * part.gemm.batch0 * part.gemm.batch1 * part.gemm.M * part.gemm.N * (part.gemm.K + (part.dual ? part.gemm2.K : 0));
      break;
    case Step::Conv: {
      kind = "conv";
      double macs = (double)s.conv.N * s.conv.O * (s.conv.C / s.conv.featureGroups);
      for (int d = 0; d < s.conv.nsp; ++d) macs *= (double)s.conv.out[d] * s.conv.k[d];
      flops = 2.0 * macs;
      break;
    }
    case Step::ScatterRows: kind = "scatter"; bytes = (double)s.scatter.numUpdates * s.scatter.rowElems * 4; break;
    case Step::Copy: kind = "copy"; bytes = 2.0 * s.bytes; break;
    default: break;
  }
  bool doTime = !kind.empty() && timedCall_ && timed(kind);
  static const bool detail = getenv("MI355X_TIMING_DETAIL") != nullptr;   // one statistics row per step label
  if (doTime && detail) kind += ":" + s.label;
  mi355_event_t ea = nullptr, eb = nullptr;
  int kernelLaunches = 1;   // launches of a Kernel step between its two events
  if (doTime) {
    ea = getEvent();
    eb = getEvent();
    mi355_event_record(ea, st);
  }
  switch (s.kind) {
    case Step::Kernel: {
      void* ptrs[256];
      void* argv[256];
      size_t n = s.args.size();
      if (n > 256) throw RuntimeError("fused kernel with more than 256 arguments");
      for (size_t i = 0; i < n; ++i) { ptrs[i] = resolve(s.args[i], in, out); argv[i] = &ptrs[i]; }
      // A timed fused kernel may be launched several times between its two events, which spreads the cost of the
      // event pair over the launches.  That leaves the result unchanged only for a kernel that is a pure function
      // of its inputs: one that writes a buffer another of its arguments reads (a loop carry updated in place,
      // x = f(x)) is launched once.
      int launches = doTime ? timingRepeat_ : 1;
      if (launches > 1) {
        for (size_t i = 0; i < n && launches > 1; ++i) {
          if (i >= s.argWrites.size() || !s.argWrites[i]) continue;
          for (size_t j = 0; j < n; ++j)
            if (j != i && ptrs[j] == ptrs[i]) { launches = 1; break; }
        }
      }
      kernelLaunches = launches;
      const int sets = launches > 1 ? (int)shadows_.size() + 1 : 1;
      for (int r = 0; r < launches; ++r) {
        if (sets > 1)
          for (size_t i = 0; i < n; ++i) ptrs[i] = resolveIn(s.args[i], r % sets, in, out);
        check(mi355_launch((mi355_function_t)prog_->kernels[s.kernel].function, s.grid, s.block, argv, (int)n, st), s.label.c_str());
      }
      break;
    }
    case Step::Gemm: {
      mi355_gemm_desc d = toAbi(s.gemm);
      const void* bias = s.bias.kind == BufRef::None ? nullptr : resolve(s.bias, in, out);
      const void* addend = s.addend.kind == BufRef::None ? nullptr : resolve(s.addend, in, out);
      if (s.dual || addend) {
        mi355_gemm_desc d2;
        if (s.dual) d2 = toAbi(s.gemm2);
        check(mi355_gemm_small_sum(&d, resolve(s.args[0], in, out), resolve(s.args[1], in, out), s.dual ? &d2 : nullptr,
                                   s.dual ? resolve(s.args[3], in, out) : nullptr, s.dual ? resolve(s.args[4], in, out) : nullptr,
                                   resolve(s.args[2], in, out), bias, addend, st), "gemm (small products summed)");
        break;
      }
      void* ws = s.args.size() > 3 ? resolve(s.args[3], in, out) : nullptr;
      check(mi355_gemm(&d, resolve(s.args[0], in, out), resolve(s.args[1], in, out), resolve(s.args[2], in, out), bias, ws,
                       (size_t)s.workspaceBytes, st), "gemm");
      break;
    }
    case Step::Attention: {
      mi355_attention_desc d = toAbi(s.attn);
      const void* mask = s.args.size() > 4 ? resolve(s.args[4], in, out) : nullptr;
      int r = mi355_attention(&d, resolve(s.args[0], in, out), resolve(s.args[1], in, out), resolve(s.args[2], in, out), mask,
                              resolve(s.args[3], in, out), st);
      if (r < 0) throw RuntimeError("attention: operands are not aligned as planned");
      check(r, "attention");
      break;
    }
    case Step::GemmGroup: {
      const int n = (int)s.parts.size();
      mi355_gemm_desc d1[4], d2[4];
      const mi355_gemm_desc *p1[4], *p2[4];
      const void *a1[4], *b1[4], *a2[4], *b2[4], *bias[4], *addend[4];
      void* c[4];
      if (n > 4) throw RuntimeError("gemm group of more than 4 products");
      for (int i = 0; i < n; ++i) {
        const Step& part = s.parts[(size_t)i];
        d1[i] = toAbi(part.gemm);
        p1[i] = &d1[i];
        a1[i] = resolve(part.args[0], in, out); b1[i] = resolve(part.args[1], in, out); c[i] = resolve(part.args[2], in, out);
        if (part.dual) {
          d2[i] = toAbi(part.gemm2);
          p2[i] = &d2[i];
          a2[i] = resolve(part.args[3], in, out); b2[i] = resolve(part.args[4], in, out);
        } else {
          p2[i] = nullptr; a2[i] = nullptr; b2[i] = nullptr;
        }
        bias[i] = part.bias.kind == BufRef::None ? nullptr : resolve(part.bias, in, out);
        addend[i] = part.addend.kind == BufRef::None ? nullptr : resolve(part.addend, in, out);
      }
      check(mi355_gemm_small_group(n, p1, a1, b1, p2, a2, b2, c, bias, addend, st), "gemm group");
      break;
    }
    case Step::Conv: {
      mi355_conv_desc d = toAbi(s.conv);
      void* ws = s.workspaceBytes > 0 && s.args.size() > 3 ? resolve(s.args[3], in, out) : nullptr;
      float* statSum = s.statsArg >= 0 ? (float*)resolve(s.args[(size_t)s.statsArg], in, out) : nullptr;
      float* statSq = s.statsArg >= 0 ? (float*)resolve(s.args[(size_t)s.statsArg + 1], in, out) : nullptr;
      check(mi355_conv_stats(&d, resolve(s.args[0], in, out), resolve(s.args[1], in, out), resolve(s.args[2], in, out), ws,
                             (size_t)s.workspaceBytes, statSum, statSq, st), "convolution");
      break;
    }
    case Step::ScatterRows: {
      mi355_scatter_desc d;
      d.numUpdates = s.scatter.numUpdates; d.rowElems = s.scatter.rowElems; d.operandRows = s.scatter.operandRows;
      d.kind = s.scatter.kind;
      d.dtype = dtypeCode(s.scatter.type);
      d.index_bytes = (int)dtypeSize(s.scatter.indexType);
      if ((size_t)s.workspaceBytes < mi355_scatter_workspace_bytes(d.numUpdates))
        throw RuntimeError("internal: scatter workspace is smaller than the kernel needs");
      const int rc = mi355_scatter_rows_fill(&d, resolve(s.args[0], in, out), resolve(s.args[1], in, out), resolve(s.args[2], in, out),
                                             resolve(s.args[3], in, out), s.scatter.fill ? 1 : 0, s.scatter.fillBits, st);
      if (rc == MI355_SCATTER_GRID_TOO_LARGE) throw RuntimeError("scatter: rows this long or updates this many need more workgroups than one launch holds");
      check(rc, "scatter");
      break;
    }
    case Step::Copy: {
      mi355_copy_cond cond;
      const mi355_copy_cond* pc = nullptr;
      if (s.condMode != 0) {
        cond.flag = resolve(s.condBuf, in, out);
        cond.mode = s.condMode;
        cond.index_bytes = s.condType == DType::Pred ? 0 : (int)dtypeSize(s.condType);
        cond.want = s.condWant;
        cond.count = s.condCount;
        pc = &cond;
      }
      if (!s.copyBytes.empty()) {
        const void* srcs[16];
        void* dsts[16];
        size_t sizes[16];
        size_t n = s.copyBytes.size();
        for (size_t i = 0; i < n; ++i) {
          srcs[i] = resolve(s.args[2 * i], in, out);
          dsts[i] = resolve(s.args[2 * i + 1], in, out);
          sizes[i] = (size_t)s.copyBytes[i];
        }
        check(mi355_copy_multi_if((int)n, dsts, srcs, sizes, pc, st), "copy");
        break;
      }
      if (pc) {
        const void* src1 = resolve(s.src, in, out);
        void* dst1 = resolve(s.dst, in, out);
        size_t size1 = (size_t)s.bytes;
        check(mi355_copy_multi_if(1, &dst1, &src1, &size1, pc, st), "conditional copy");
        break;
      }
      check(mi355_copy(resolve(s.dst, in, out), resolve(s.src, in, out), (size_t)s.bytes, st), "copy");
      break;
    }
    case Step::Fill: break;
    case Step::FlagInit:
      check(mi355_flag_init(resolve(s.flagBuf, in, out), s.parentFlag.kind == BufRef::None ? nullptr : resolve(s.parentFlag, in, out), st), "loop flag");
      break;
    case Step::FlagAnd:
      check(mi355_flag_and(resolve(s.flagBuf, in, out), resolve(s.predBuf, in, out), st), "loop flag update");
      break;
    case Step::While: {
      if (s.tripCount >= 0) {
        // counted loop: the trip count is known, iterations are queued back to back with no host round trip
        runCountedLoop(s, in, out);
      } else if (s.flagBuf.kind != BufRef::None) {
        runDeviceLoop(s, in, out);
      } else {
        unsigned char* flag = (unsigned char*)dev.pinnedScratch();
        while (true) {
          runPlan(*s.cond, in, out);
          check(mi355_memcpy_d2h(flag, resolve(s.predBuf, in, out), 1, st), "predicate read-back");
          dev.sync();
          if (!*flag) break;
          runPlan(*s.bodies[0], in, out);
        }
      }
      break;
    }
    case Step::Case: {
      if (s.predicated) {
        // every branch runs; only the selected one's result copies take effect (decided on the device)
        for (auto& b : s.bodies) runPlan(*b, in, out);
        break;
      }
      long long idx = 0;
      size_t sz = dtypeSize(s.predType);
      void* host = dev.pinnedScratch();
      check(mi355_memcpy_d2h(host, resolve(s.predBuf, in, out), sz, st), "branch index read-back");
      dev.sync();
      if (s.predType == DType::Pred) idx = *(unsigned char*)host ? 1 : 0;
      else if (sz == 4) idx = *(int*)host;
      else if (sz == 8) idx = *(long long*)host;
      else if (sz == 1) idx = *(signed char*)host;
      else idx = *(short*)host;
      long long nb = (long long)s.bodies.size();
      // out-of-range selects the last branch (reference: ops/control_flow.cc:672-675)
      if (idx < 0 || idx >= nb) idx = nb - 1;
      runPlan(*s.bodies[(size_t)idx], in, out);
      break;
    }
  }
  if (doTime) {
    mi355_event_record(eb, st);
    const double launches = (double)kernelLaunches;
    pending_.push_back({ea, eb, kind, flops * launches, bytes * launches, launches});
    if (pending_.size() > 20000) resolvePending();
  }
}

bool Executable::capturable(const Plan& p) {
  auto it = capturable_.find(&p);
  if (it != capturable_.end()) return it->second;
  bool ok = true;
  for (auto& s : p.steps) {
    switch (s.kind) {
      case Step::Kernel: case Step::Gemm: case Step::GemmGroup: case Step::Attention: case Step::Conv: case Step::ScatterRows: case Step::Copy: case Step::Fill:
      case Step::FlagInit: case Step::FlagAnd: break;
      case Step::While: ok = ok && s.tripCount >= 0 && capturable(*s.bodies[0]); break;   // dynamic loops read a flag back on the host
      case Step::Case:
        ok = ok && s.predicated;
        for (auto& b : s.bodies) ok = ok && capturable(*b);
        break;
      default: ok = false; break;
    }
  }
  capturable_[&p] = ok;
  return ok;
}

// Iterations of a counted loop are identical launch sequences over fixed addresses (the counter
// and the carries live in the arena), so after one eager iteration the body is captured into a
// graph holding several iterations and replayed; the host then issues one launch per replay
// instead of one per kernel.
void Executable::runCountedLoop(const Step& s, const std::vector<DeviceBuffer*>& in, const std::vector<void*>& out) {
  replayIterations(s, false, s.tripCount, in, out);
}

// A loop whose trip count depends on data.  Iterations are queued in chunks (4, 4, 8, 16, 32, 64, 64 ...) with no host round trip
// inside a chunk: each iteration evaluates the condition, folds it into the loop's flag on the device, runs the body
// into temporaries and commits the carries only while the flag is set, so iterations queued past the end change
// nothing.  The host reads the flag once per chunk.  At most as many iterations run past the end as ran before it.
void Executable::runDeviceLoop(const Step& s, const std::vector<DeviceBuffer*>& in, const std::vector<void*>& out) {
  Device& dev = Device::get();
  int* flag = (int*)dev.pinnedScratch();
  // The first chunk is as long as the loop ran the last time (plus the evaluation of the condition that ends it):
  // a loop that repeats its trip count from call to call then costs one round trip and queues nothing past its end.
  int64_t& last = lastTrips_[&s];
  int64_t chunk = last > 0 ? std::min<int64_t>(last + 1, 256) : 4;
  while (true) {
    replayIterations(s, true, chunk, in, out);
    check(mi355_memcpy_d2h(flag, resolve(s.flagBuf, in, out), 8, dev.stream()), "loop flag read-back");
    dev.sync();
    ++loopSyncs_;
    if (!flag[0]) break;
    chunk = std::min<int64_t>(std::max<int64_t>(4, (int64_t)flag[1]), 64);   // as many again as have run, 64 at most
  }
  last = flag[1];
}

// `count` iterations of a loop: the body alone (counted loops) or condition + body (loops kept alive by a device flag).
void Executable::replayIterations(const Step& s, bool withCond, int64_t trip, const std::vector<DeviceBuffer*>& in, const std::vector<void*>& out) {
  Device& dev = Device::get();
  const Plan& body = *s.bodies[0];
  // A loop whose counter the host follows gives every iteration its own addresses (hostIteration_ selects them), so its
  // graph holds all iterations after the first and is launched once.
  const bool counted = s.hostCounter;
  int64_t iteration = 0;
  auto runOne = [&]() {
    if (counted) hostIteration_ = iteration++;
    if (withCond) runPlan(*s.cond, in, out);
    runPlan(body, in, out);
  };
  struct RestoreIteration { int64_t& v; int64_t was; ~RestoreIteration() { v = was; } } restoreIteration{hostIteration_, hostIteration_};   // (an inner loop leaves the outer loop's iteration as it found it)
  const size_t unitSteps = body.steps.size() + (withCond ? s.cond->steps.size() : 0);
  const int64_t nodeLimit = counted ? 8192 : 1024;
  const bool graphOk = useGraphs_ && !capturing_ && timingKinds_.empty() && trip >= (withCond ? 16 : 4) && unitSteps > 0 && capturable(body) &&
                       (!withCond || capturable(*s.cond)) && (!counted || (trip - 1) * (int64_t)unitSteps <= nodeLimit);
  if (!graphOk) {
    for (int64_t i = 0; i < trip; ++i) runOne();
    return;
  }
  if (!withCond) runOne();   // first iteration eagerly: finishes lazy one-time set-up outside the capture
  LoopGraphs& lgs = loopGraphs_[&s];
  if (!lgs.scanned) {
    std::function<void(const Plan&)> scan = [&](const Plan& p) {
      auto add = [&](const BufRef& b) { if (b.kind == BufRef::Param || b.kind == BufRef::Output) lgs.external.push_back(b); };
      for (auto& st : p.steps) {
        for (auto& a : st.args) add(a);
        for (auto& part : st.parts) { for (auto& a : part.args) add(a); add(part.bias); add(part.addend); }
        add(st.src); add(st.dst); add(st.predBuf); add(st.bias); add(st.addend);
        if (st.cond) scan(*st.cond);
        for (auto& b : st.bodies) scan(*b);
      }
    };
    scan(body);
    if (withCond) scan(*s.cond);
    lgs.scanned = true;
  }
  uint64_t sig = 1469598103934665603ull;
  for (auto& b : lgs.external) sig = (sig ^ (uint64_t)(uintptr_t)resolve(b, in, out)) * 1099511628211ull;
  LoopGraph* hit = nullptr;
  for (auto& e : lgs.entries) if (e.exec && e.signature == sig) hit = &e;
  if (!hit) {
    if (lgs.entries.size() < 4) {
      lgs.entries.emplace_back();
      hit = &lgs.entries.back();
    } else {
      hit = &lgs.entries[0];
      for (auto& e : lgs.entries) if (e.lastUse < hit->lastUse) hit = &e;
      // replays of the evicted graph may still be queued
      dev.sync();
      mi355_graph_destroy(hit->exec);
      hit->exec = nullptr;
    }
    // a flag-driven loop is replayed in sub-chunks of 16 iterations, so that one graph serves whatever length the next chunk has
    const int64_t per = counted ? trip - 1 : std::max<int64_t>(1, std::min<int64_t>(withCond ? 16 : trip - 1, 1024 / (int64_t)unitSteps));
    mi355_stream_t st = dev.stream();
    check(mi355_capture_begin(st), "graph capture");
    capturing_ = true;
    try {
      iteration = 1;
      for (int64_t i = 0; i < per; ++i) runOne();
    } catch (...) {
      capturing_ = false;
      mi355_graph_t dead = nullptr;
      int n = 0;
      if (mi355_capture_end(st, &dead, &n) == 0 && dead) mi355_graph_destroy(dead);
      throw;
    }
    capturing_ = false;
    int nodes = 0;
    check(mi355_capture_end(st, &hit->exec, &nodes), "graph instantiate");
    hit->signature = sig;
    hit->itersPerLaunch = per;
    static const bool verbose = getenv("MI355X_VERBOSE") != nullptr;
    if (verbose) fprintf(stderr, "[mi355x] loop body captured: %lld iteration(s), %d graph nodes\n", (long long)per, nodes);
  }
  hit->lastUse = ++graphClock_;
  LoopGraph& lg = *hit;
  int64_t left = withCond ? trip : trip - 1;
  for (; left >= lg.itersPerLaunch; left -= lg.itersPerLaunch) check(mi355_graph_launch(lg.exec, dev.stream()), "graph launch");
  for (; left > 0; --left) runOne();
}

void Executable::runPlan(const Plan& plan, const std::vector<DeviceBuffer*>& in, const std::vector<void*>& out) {
  // Forked steps run on the second stream: it waits for everything enqueued so far, and the step that first needs the
  // result (or the end of the plan) makes the main stream wait for it.  A call whose steps are being timed runs
  // everything in order on the main stream, so that the step times stay those of the kernels alone.
  static const bool forking = !getenv("MI355X_SECOND_STREAM") || atoi(getenv("MI355X_SECOND_STREAM")) != 0;
  if (plan.numForks == 0 || !forking || !forkingAllowed_ || (timedCall_ && !timingKinds_.empty())) {
    for (auto& s : plan.steps) runStep(s, in, out);
    return;
  }
  Device& dev = Device::get();
  if (!sideStream_) check(mi355_stream_create(&sideStream_), "second stream");
  while (forkStart_.size() < (size_t)plan.numForks) {
    mi355_event_t a = nullptr, b = nullptr;
    check(mi355_event_create(&a, 0), "event");
    check(mi355_event_create(&b, 0), "event");
    forkStart_.push_back(a);
    forkDone_.push_back(b);
  }
  std::vector<char> pending((size_t)plan.numForks, 0);
  bool sideDirty = false;     // something was enqueued on the second stream that the main stream has not joined yet
  try {
    for (auto& s : plan.steps) {
      for (int id : s.joins) {
        if (!pending[(size_t)id]) continue;
        check(mi355_stream_wait_event(dev.stream(), forkDone_[(size_t)id]), "join");
        pending[(size_t)id] = 0;
      }
      if (s.forkId < 0) { runStep(s, in, out); continue; }
      const size_t id = (size_t)s.forkId;
      check(mi355_event_record(forkStart_[id], dev.stream()), "fork");
      check(mi355_stream_wait_event(sideStream_, forkStart_[id]), "fork");
      streamOverride_ = sideStream_;
      sideDirty = true;
      try { runStep(s, in, out); } catch (...) { streamOverride_ = nullptr; throw; }
      streamOverride_ = nullptr;
      check(mi355_event_record(forkDone_[id], sideStream_), "fork");
      pending[id] = 1;
    }
    for (size_t id = 0; id < pending.size(); ++id)
      if (pending[id]) check(mi355_stream_wait_event(dev.stream(), forkDone_[id]), "join");
  } catch (...) {
    // Invariant the allocator relies on: side-stream work is always joined before execute returns or throws, because
    // blocks released afterwards are recycled on the assumption that the main stream orders every use of them.  On
    // the error path the host waits for the second stream (the failing step may have left it without a done event).
    if (sideDirty) mi355_stream_sync(sideStream_);
    throw;
  }
}

// One graph launch for the whole plan, when this call's buffer addresses have been seen before.  False: the caller
// runs the plan launch by launch.
bool Executable::runPlanFromGraph(const std::vector<DeviceBuffer*>& in, const std::vector<void*>& out) {
  static const bool forkInside = !getenv("MI355X_PLAN_GRAPH_FORKS") || atoi(getenv("MI355X_PLAN_GRAPH_FORKS")) != 0;
  if (!planGraphsOn_ || !useGraphs_ || capturing_ || planGraphState_ == 0) return false;
  if (timedCall_ && !timingKinds_.empty()) return false;       // a timed call brackets its steps with events
  const Plan& plan = prog_->plan;
  if (planGraphState_ < 0) {
    bool ok = plan.steps.size() >= 2 && capturable(plan);
    for (auto& s : plan.steps) if (s.kind == Step::While || s.kind == Step::Case) ok = false;   // loops replay graphs of their own
    planGraphState_ = ok ? 1 : 0;
    if (!ok) return false;
  }
  Device& dev = Device::get();
  uint64_t sig = 1469598103934665603ull;
  for (auto* b : in) sig = (sig ^ (uint64_t)(uintptr_t)b->ptr) * 1099511628211ull;
  for (auto* p : out) sig = (sig ^ (uint64_t)(uintptr_t)p) * 1099511628211ull;
  PlanGraph* hit = nullptr;
  for (auto& g : planGraphs_) if (g.exec && g.signature == sig) hit = &g;
  if (!hit) {
    bool seen = false;
    for (auto v : seenSignatures_) seen = seen || v == sig;
    if (!seen) {
      if (seenSignatures_.size() >= 8) seenSignatures_.erase(seenSignatures_.begin());
      seenSignatures_.push_back(sig);
      if (++planGraphMisses_ >= 64 && planGraphLaunches_ == 0) planGraphState_ = 0;   // addresses never repeat here
      return false;
    }
    if (planGraphs_.size() < 4) {
      planGraphs_.emplace_back();
      hit = &planGraphs_.back();
    } else {
      hit = &planGraphs_[0];
      for (auto& g : planGraphs_) if (g.lastUse < hit->lastUse) hit = &g;
      dev.sync();                        // replays of the evicted graph may still be queued
      mi355_graph_destroy(hit->exec);
      hit->exec = nullptr;
    }
    mi355_stream_t st = dev.stream();
    const bool forkWas = forkingAllowed_;
    forkingAllowed_ = forkInside;
    check(mi355_capture_begin(st), "graph capture");
    capturing_ = true;
    try {
      runPlan(plan, in, out);
    } catch (...) {
      capturing_ = false;
      forkingAllowed_ = forkWas;
      mi355_graph_t dead = nullptr;
      int n = 0;
      if (mi355_capture_end(st, &dead, &n) == 0 && dead) mi355_graph_destroy(dead);
      planGraphState_ = 0;
      throw;
    }
    capturing_ = false;
    forkingAllowed_ = forkWas;
    int nodes = 0;
    check(mi355_capture_end(st, &hit->exec, &nodes), "graph instantiate");
    hit->signature = sig;
    if (getenv("MI355X_VERBOSE")) fprintf(stderr, "[mi355x] whole plan captured: %zu steps, %d graph nodes\n", plan.steps.size(), nodes);
  }
  hit->lastUse = ++graphClock_;
  check(mi355_graph_launch(hit->exec, dev.stream()), "graph launch");
  ++planGraphLaunches_;
  return true;
}

std::vector<std::shared_ptr<DeviceBuffer>> Executable::execute(const std::vector<DeviceBuffer*>& inputs, const std::vector<bool>* mayDonate) {
  std::lock_guard<std::mutex> lk(mu_);
  Device& dev = Device::get();
  if (inputs.size() != prog_->paramTypes.size())
    throw RuntimeError("execute: expected " + std::to_string(prog_->paramTypes.size()) + " arguments, got " + std::to_string(inputs.size()));
  for (size_t i = 0; i < inputs.size(); ++i) {
    if (!inputs[i] || inputs[i]->deleted || !inputs[i]->ptr) throw RuntimeError("execute: argument " + std::to_string(i) + " is null or deleted");
    if (!(inputs[i]->type == prog_->paramTypes[i]))
      throw RuntimeError("execute: argument " + std::to_string(i) + " has type " + inputs[i]->type.str() + ", executable expects " + prog_->paramTypes[i].str());
  }
  std::vector<std::shared_ptr<DeviceBuffer>> outs;
  std::vector<void*> outPtrs;
  for (auto& o : prog_->outputs) {
    auto b = std::make_shared<DeviceBuffer>();
    b->type = o.type;
    b->ptr = dev.alloc(std::max<size_t>(o.type.bytes(), 4));
    outPtrs.push_back(b->ptr);
    outs.push_back(std::move(b));
  }
  timedCall_ = (executeCount_++ % timingEvery_) == 0;
  if (timedCall_ && timingRepeat_ > 1 && !timingKinds_.empty()) prepareShadows(inputs);
  if (!runPlanFromGraph(inputs, outPtrs)) runPlan(prog_->plan, inputs, outPtrs);
  if (mayDonate) {
    // (released last to first: the next call's results, allocated first to last, then take these blocks in order)
    for (size_t i = std::min(inputs.size(), prog_->paramDonation.size()); i-- > 0;) {
      if (prog_->paramDonation[i] == -1 || i >= mayDonate->size() || !(*mayDonate)[i]) continue;
      bool again = false;   // the same buffer passed for another argument stays alive
      for (size_t j = 0; j < inputs.size(); ++j) if (j != i && inputs[j] == inputs[i]) again = true;
      if (again) continue;
      dev.release(inputs[i]->ptr);
      inputs[i]->ptr = nullptr;
      inputs[i]->deleted = true;
    }
  }
  return outs;
}

}  // namespace mi355
