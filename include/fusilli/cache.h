// On-disk cache files of a compiled graph.
//
// Same contract as the reference's support/cache.h:71-250: files live under
// ${FUSILLI_CACHE_DIR or HOME}/.cache/fusilli/<graphName>/<fileName>; a
// CacheFile created with remove = true deletes its file (and the graph's
// directory once empty) when the object goes out of scope; open() fails for a
// file that does not exist.  What the files hold differs: a textual
// description of the planned graph, the key of the planner that produced the
// artifact, and the serialised plan (plan.h) where the reference keeps MLIR,
// the iree-compile command line and a .vmfb.
#ifndef FUSILLI_CACHE_H
#define FUSILLI_CACHE_H

#include <cstdlib>
#include <filesystem>
#include <fstream>
#include <span>
#include <sstream>
#include <string>
#include <vector>

#include "errors.h"

namespace fusilli {

class CacheFile {
public:
  std::filesystem::path path;

  // Creates (or truncates) the file.
  static ErrorOr<CacheFile> create(const std::string &graphName,
                                   const std::string &fileName, bool remove) {
    std::filesystem::path p = getPath(graphName, fileName);
    std::error_code ec;
    std::filesystem::create_directories(p.parent_path(), ec);
    FUSILLI_RETURN_ERROR_IF(ec, ErrorCode::FileSystemFailure,
                            "Failed to create cache directory: " +
                                p.parent_path().string() + " - " + ec.message());
    std::ofstream file(p, std::ios::binary | std::ios::trunc);
    FUSILLI_RETURN_ERROR_IF(!file.is_open(), ErrorCode::FileSystemFailure,
                            "Failed to create file: " + p.string());
    file.close();
    return ok(CacheFile(std::move(p), remove));
  }

  // Opens an existing file (never removed by the returned object).
  static ErrorOr<CacheFile> open(const std::string &graphName,
                                 const std::string &fileName) {
    std::filesystem::path p = getPath(graphName, fileName);
    FUSILLI_RETURN_ERROR_IF(!std::filesystem::exists(p),
                            ErrorCode::FileSystemFailure,
                            "File does not exist: " + p.string());
    return ok(CacheFile(std::move(p), /*remove=*/false));
  }

  // ${FUSILLI_CACHE_DIR}/.cache/fusilli, else ${HOME}/.cache/fusilli, else
  // the system's temporary directory.
  static std::filesystem::path getCacheDir() {
    const char *dir = std::getenv("FUSILLI_CACHE_DIR");
    if (!dir || !*dir)
      dir = std::getenv("HOME");
    std::filesystem::path base;
    if (dir && *dir) {
      base = dir;
    } else {
      std::error_code ec;
      base = std::filesystem::temp_directory_path(ec);
      if (ec)
        base = ".";
    }
    return base / ".cache" / "fusilli";
  }

  // Graph names become directory names: anything but [A-Za-z0-9._-] is
  // replaced, so a name cannot leave the cache directory.
  static std::filesystem::path getPath(const std::string &graphName,
                                       const std::string &fileName) {
    std::string safe = graphName;
    for (char &c : safe) {
      const bool keep = (c >= 'a' && c <= 'z') || (c >= 'A' && c <= 'Z') ||
                        (c >= '0' && c <= '9') || c == '_' || c == '-' || c == '.';
      if (!keep)
        c = '_';
    }
    if (safe.empty() || safe == "." || safe == "..")
      safe = "_" + safe;
    return getCacheDir() / safe / fileName;
  }

  ErrorObject write(const std::string &content) {
    return write(std::span<const uint8_t>(
        reinterpret_cast<const uint8_t *>(content.data()), content.size()));
  }
  ErrorObject write(std::span<const uint8_t> bytes) {
    std::ofstream file(path, std::ios::binary | std::ios::trunc);
    FUSILLI_RETURN_ERROR_IF(!file.is_open(), ErrorCode::FileSystemFailure,
                            "Failed to open file: " + path.string());
    file.write(reinterpret_cast<const char *>(bytes.data()),
               static_cast<std::streamsize>(bytes.size()));
    FUSILLI_RETURN_ERROR_IF(!file.good(), ErrorCode::FileSystemFailure,
                            "Failed to write file: " + path.string());
    return ok();
  }
  ErrorOr<std::string> read() const {
    std::ifstream file(path, std::ios::binary);
    FUSILLI_RETURN_ERROR_IF(!file.is_open(), ErrorCode::FileSystemFailure,
                            "Failed to open file: " + path.string());
    std::ostringstream ss;
    ss << file.rdbuf();
    return ok(ss.str());
  }
  ErrorOr<std::vector<uint8_t>> readBytes() const {
    FUSILLI_ASSIGN_OR_RETURN(std::string s, read());
    return ok(std::vector<uint8_t>(s.begin(), s.end()));
  }

  CacheFile(const CacheFile &) = delete;
  CacheFile &operator=(const CacheFile &) = delete;
  CacheFile(CacheFile &&other) noexcept
      : path(std::move(other.path)), remove_(other.remove_) {
    other.remove_ = false;
    other.path.clear();
  }
  CacheFile &operator=(CacheFile &&other) noexcept {
    if (this != &other) {
      cleanup();
      path = std::move(other.path);
      remove_ = other.remove_;
      other.remove_ = false;
      other.path.clear();
    }
    return *this;
  }
  ~CacheFile() { cleanup(); }

private:
  CacheFile(std::filesystem::path p, bool remove)
      : path(std::move(p)), remove_(remove) {}

  void cleanup() noexcept {
    if (!remove_ || path.empty())
      return;
    std::error_code ec;
    std::filesystem::remove(path, ec);
    // the graph's directory, once its last file is gone
    const std::filesystem::path dir = path.parent_path();
    if (std::filesystem::is_directory(dir, ec) &&
        std::filesystem::is_empty(dir, ec))
      std::filesystem::remove(dir, ec);
    remove_ = false;
  }

  bool remove_ = false;
};

// The files of one compiled graph (reference support/cache.h:303-335).
struct CachedAssets {
  CacheFile input;      // description of the planned graph
  CacheFile output;     // the artifact
  CacheFile command;    // planner key (backend, plan format)
  CacheFile statistics; // JSON: dispatch count and workspace bytes of the plan
                        // (the reference keeps iree-compile's statistics here)
};

// (reference support/cache.h:306-312)
enum class CachedAssetsType { Input, Output, Command, Statistics };

inline constexpr const char *kCacheInputFileName = "fusilli_plan_input.txt";
inline constexpr const char *kCacheOutputFileName = "fusilli_plan_output.bin";
inline constexpr const char *kCacheCommandFileName = "fusilli_plan_command.txt";
inline constexpr const char *kCacheStatisticsFileName = "fusilli_plan_statistics.json";

} // namespace fusilli

#endif // FUSILLI_CACHE_H
