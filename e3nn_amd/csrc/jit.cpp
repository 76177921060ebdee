// Kernel specialisation: source assembly, on-disk code-object cache, compiler driver.
//
// A specialised kernel = generated constexpr tables (one instruction set) + a fixed
// hand-written device template.  The code object is compiled once with the system HIP
// compiler and kept under the cache directory, keyed by a hash of the full source text,
// the compiler flags and the compiler's identity (what it prints for --version), so
// identical instruction sets never compile twice and a compiler upgrade never reuses
// code objects of the old one.
#include <atomic>
#include <dlfcn.h>
#include <fcntl.h>
#include <spawn.h>
#include <sys/stat.h>
#include <sys/wait.h>
#include <unistd.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <mutex>
#include <sstream>

#include "e3x_internal.h"
#include "jit.h"

extern char** environ;

namespace e3x {

static const char* kFlags[] = {"--genco", "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature",
                               "-Xclang", "-packed-fp32-ops", "-ffp-contract=fast", "-Wno-unused-value"};

static uint64_t fnv1a(const std::string& s, uint64_t h = 1469598103934665603ULL) {
  for (unsigned char c : s) {
    h ^= c;
    h *= 1099511628211ULL;
  }
  return h;
}

static bool file_exists(const std::string& p) {
  struct stat st;
  return ::stat(p.c_str(), &st) == 0 && st.st_size > 0;
}

std::string cache_dir() {
  if (const char* env = std::getenv("E3X_KERNEL_CACHE")) return env;
  Dl_info info;
  if (dladdr((void*)&cache_dir, &info) && info.dli_fname) {
    std::string lib = info.dli_fname;
    size_t s = lib.rfind('/');
    std::string dir = s == std::string::npos ? "." : lib.substr(0, s);
    return dir + "/../kernel_cache";
  }
  return "./kernel_cache";
}

static std::string find_compiler() {
  if (const char* env = std::getenv("E3X_HIPCC")) return env;
  if (file_exists("/opt/rocm/bin/hipcc")) return "/opt/rocm/bin/hipcc";
  return "hipcc";
}

// What identifies the compiler in the cache key: $E3X_COMPILER_ID when set (a deployment that ships a prebuilt cache
// and no compiler names the one that built it), else the first two lines of `<compiler> --version` (HIP version and
// clang version with its commit).  The compiler is asked once per installation, not per process: the answer is kept
// in <cache>/compiler_id behind a signature of the installation (resolved paths and sizes of the driver and of the
// clang++ it runs), and a process whose compiler still has that signature reads it from there without starting a
// child process.
static std::string installation_signature(const std::string& cc) {
  std::string sig;
  auto add = [&](const std::string& p) {
    char real[4096];
    struct stat st;
    if (::realpath(p.c_str(), real) && ::stat(real, &st) == 0) sig += std::string(real) + ":" + std::to_string((long long)st.st_size) + ";";
  };
  add(cc);
  char real[4096];
  if (::realpath(cc.c_str(), real)) {
    std::string dir = real;
    size_t s = dir.rfind('/');
    if (s != std::string::npos) add(dir.substr(0, s) + "/../lib/llvm/bin/clang++");
  }
  return sig.empty() ? cc : sig;
}

static const std::string& compiler_identity(const std::string& cc) {
  static std::once_flag once;
  static std::string id;
  std::call_once(once, [&] {
    if (const char* env = std::getenv("E3X_COMPILER_ID")) {
      id = env;
      return;
    }
    const std::string sig = installation_signature(cc), note = cache_dir() + "/compiler_id";
    {
      std::ifstream f(note);
      std::string first;
      if (f && std::getline(f, first) && first == sig) {
        std::stringstream rest;
        rest << f.rdbuf();
        id = rest.str();
        if (!id.empty()) return;
      }
    }
    std::string cmd;
    for (char c : cc) cmd += (c == '\'') ? std::string("'\\''") : std::string(1, c);
    cmd = "'" + cmd + "' --version 2>/dev/null";
    if (FILE* f = ::popen(cmd.c_str(), "r")) {
      char line[512];
      for (int n = 0; n < 2 && std::fgets(line, sizeof(line), f); n++) id += line;
      ::pclose(f);
    }
    if (id.empty()) return;  // no compiler to ask: keys carry no compiler identity and nothing can be compiled anyway
    ::mkdir(cache_dir().c_str(), 0755);
    char tag[64];
    std::snprintf(tag, sizeof(tag), ".tmp%d", (int)getpid());
    std::ofstream f(note + tag);
    if (f) {
      f << sig << "\n" << id;
      f.close();
      std::rename((note + tag).c_str(), note.c_str());
    }
  });
  return id;
}

int get_code_object(const std::string& family, const std::string& source, std::string* key_out,
                    std::string* path_out) {
  std::string flags;
  for (const char* f : kFlags) flags += std::string(f) + " ";
  const std::string cc = find_compiler();
  const uint64_t h1 = fnv1a(source), h2 = fnv1a(compiler_identity(cc) + flags + source, 0x9e3779b97f4a7c15ULL);
  char key[64];
  std::snprintf(key, sizeof(key), "%s_%016llx%08llx", family.c_str(), (unsigned long long)h1,
                (unsigned long long)(h2 & 0xffffffffULL));
  const std::string dir = cache_dir();
  const std::string base = dir + "/" + key;
  *key_out = key;
  *path_out = base + ".hsaco";
  if (file_exists(*path_out)) return E3X_OK;
  // a source that the compiler has rejected before (same compiler, same flags) is not compiled again: the log is kept
  const std::string failed_path = base + ".failed";
  if (file_exists(failed_path)) {
    std::ifstream lf(failed_path);
    std::stringstream ss;
    ss << lf.rdbuf();
    return fail(E3X_ERR_COMPILE, "compiling " + base + ".hip failed before (delete " + failed_path + " to try again):\n" + ss.str());
  }

  if (const char* nojit = std::getenv("E3X_NO_JIT"))
    if (nojit[0] == '1')
      return fail(E3X_ERR_COMPILE, "kernel " + std::string(key) + " is not in the cache (" + dir +
                                       ") and E3X_NO_JIT=1 forbids compiling it");
  ::mkdir(dir.c_str(), 0755);
  // Threads and processes may build the same kernel at the same time: each works on files of its own and moves
  // the results into place at the end (rename is atomic; the contents are identical whoever wins).
  static std::atomic<unsigned> serial{0};
  char tag[64];
  std::snprintf(tag, sizeof(tag), ".tmp%d_%u", (int)getpid(), serial.fetch_add(1));
  const std::string final_src = base + ".hip";
  const std::string src_path = base + tag + ".hip", log_path = base + tag + ".log", tmp_path = base + tag + ".hsaco";
  {
    std::ofstream f(src_path);
    if (!f) return fail(E3X_ERR_COMPILE, "cannot write " + src_path);
    f << source;
  }
  std::vector<std::string> args = {cc};
  for (const char* f : kFlags) args.push_back(f);
  args.push_back("-o");
  args.push_back(tmp_path);
  args.push_back(src_path);
  std::vector<char*> argv;
  for (auto& a : args) argv.push_back(const_cast<char*>(a.c_str()));
  argv.push_back(nullptr);

  posix_spawn_file_actions_t fa;
  posix_spawn_file_actions_init(&fa);
  posix_spawn_file_actions_addopen(&fa, 1, log_path.c_str(), O_WRONLY | O_CREAT | O_TRUNC, 0644);
  posix_spawn_file_actions_adddup2(&fa, 1, 2);
  pid_t pid = 0;
  int rc = posix_spawnp(&pid, cc.c_str(), &fa, nullptr, argv.data(), environ);
  posix_spawn_file_actions_destroy(&fa);
  if (rc != 0) return fail(E3X_ERR_COMPILE, "cannot start the HIP compiler '" + cc + "': " + std::strerror(rc));
  int status = 0;
  while (waitpid(pid, &status, 0) < 0) {
    if (errno != EINTR) return fail(E3X_ERR_COMPILE, "waitpid on the HIP compiler failed");
  }
  if (!WIFEXITED(status) || WEXITSTATUS(status) != 0 || !file_exists(tmp_path)) {
    std::ifstream lf(log_path);
    std::stringstream ss;
    ss << lf.rdbuf();
    std::string log = ss.str();
    if (log.size() > 2000) log = log.substr(0, 2000) + "...";
    std::rename(src_path.c_str(), final_src.c_str());  // keep the source that failed next to its key
    std::remove(log_path.c_str());
    std::remove(tmp_path.c_str());
    if (WIFEXITED(status) && WEXITSTATUS(status) == 1 && !log.empty()) {  // the compiler's verdict, not a killed or missing compiler
      std::ofstream ff(failed_path);
      ff << log;
    }
    return fail(E3X_ERR_COMPILE, "compiling " + final_src + " failed:\n" + log);
  }
  std::rename(src_path.c_str(), final_src.c_str());
  std::remove(log_path.c_str());
  if (std::rename(tmp_path.c_str(), path_out->c_str()) != 0)
    return fail(E3X_ERR_COMPILE, "cannot move the code object into the cache");
  return E3X_OK;
}

}  // namespace e3x
