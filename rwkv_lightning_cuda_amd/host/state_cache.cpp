// Session state cache: device clones (level 1) -> host copies (level 2) -> SQLite rows (level 3).
// Behaviour follows the reference's src/rwkv_state_cache.cpp: put_state :327-345, get_state :347-381,
// eviction :246-268, schema :104-130, row format :270-325, delete/list/timestamp :383-455.
// libsqlite3 is opened with dlopen so the library has no link-time dependency on it.
#include "rwkv_state_cache.hpp"

#include <dlfcn.h>

#include <ctime>
#include <stdexcept>

namespace rwkv7_server {
namespace {

using rwkv7_fast_v4::check_hip;
using rwkv7_fast_v4::DeviceBuffer;

template <typename T, typename H>
std::vector<H> download(const DeviceBuffer<T>& buf, const char* what) {
  static_assert(sizeof(T) == sizeof(H), "element sizes must match");
  std::vector<H> host(buf.n);
  if (buf.n) check_hip(rwkv_hip_memcpy_d2h(host.data(), buf.p, buf.n * sizeof(T)), what);
  return host;
}

template <typename T, typename H>
void upload(const std::vector<H>& host, DeviceBuffer<T>& buf, const char* what) {
  static_assert(sizeof(T) == sizeof(H), "element sizes must match");
  buf.resize(host.size(), what);
  if (!host.empty()) check_hip(rwkv_hip_memcpy_h2d(buf.p, host.data(), host.size() * sizeof(T)), what);
}

template <typename T>
void duplicate(const DeviceBuffer<T>& src, DeviceBuffer<T>& dst, const char* what) {
  dst.resize(src.n, what);
  if (src.n) check_hip(rwkv_hip_memcpy_d2d(dst.p, src.p, src.n * sizeof(T)), what);
}

constexpr int kSqliteOk = 0;
constexpr int kSqliteRow = 100;
constexpr int kSqliteDone = 101;
using Destructor = void (*)(void*);
const Destructor kTransient = reinterpret_cast<Destructor>(-1);  // SQLITE_TRANSIENT: sqlite copies the bytes

}  // namespace

// Run-time binding of the few sqlite3 entry points this file uses.
struct StateCacheManager::Db {
  void* lib = nullptr;
  void* handle = nullptr;  // sqlite3*

  int (*open)(const char*, void**) = nullptr;
  int (*close)(void*) = nullptr;
  int (*exec)(void*, const char*, int (*)(void*, int, char**, char**), void*, char**) = nullptr;
  void (*free_)(void*) = nullptr;
  int (*prepare)(void*, const char*, int, void**, const char**) = nullptr;
  int (*bind_text)(void*, int, const char*, int, Destructor) = nullptr;
  int (*bind_int)(void*, int, int) = nullptr;
  int (*bind_blob)(void*, int, const void*, int, Destructor) = nullptr;
  int (*bind_double)(void*, int, double) = nullptr;
  int (*step)(void*) = nullptr;
  int (*finalize)(void*) = nullptr;
  int (*column_int)(void*, int) = nullptr;
  const void* (*column_blob)(void*, int) = nullptr;
  int (*column_bytes)(void*, int) = nullptr;
  const unsigned char* (*column_text)(void*, int) = nullptr;
  double (*column_double)(void*, int) = nullptr;
  int (*changes)(void*) = nullptr;

  template <typename F>
  bool bind(F& fn, const char* name) {
    fn = reinterpret_cast<F>(dlsym(lib, name));
    return fn != nullptr;
  }

  // Returns nullptr when libsqlite3 is not installed.
  static std::shared_ptr<Db> load() {
    auto db = std::make_shared<Db>();
    for (const char* name : {"libsqlite3.so.0", "libsqlite3.so"}) {
      db->lib = dlopen(name, RTLD_NOW | RTLD_LOCAL);
      if (db->lib) break;
    }
    if (!db->lib) return nullptr;
    const bool ok = db->bind(db->open, "sqlite3_open") && db->bind(db->close, "sqlite3_close") &&
                    db->bind(db->exec, "sqlite3_exec") && db->bind(db->free_, "sqlite3_free") &&
                    db->bind(db->prepare, "sqlite3_prepare_v2") && db->bind(db->bind_text, "sqlite3_bind_text") &&
                    db->bind(db->bind_int, "sqlite3_bind_int") && db->bind(db->bind_blob, "sqlite3_bind_blob") &&
                    db->bind(db->bind_double, "sqlite3_bind_double") && db->bind(db->step, "sqlite3_step") &&
                    db->bind(db->finalize, "sqlite3_finalize") && db->bind(db->column_int, "sqlite3_column_int") &&
                    db->bind(db->column_blob, "sqlite3_column_blob") &&
                    db->bind(db->column_bytes, "sqlite3_column_bytes") &&
                    db->bind(db->column_text, "sqlite3_column_text") &&
                    db->bind(db->column_double, "sqlite3_column_double") && db->bind(db->changes, "sqlite3_changes");
    if (!ok) return nullptr;
    return db;
  }

  ~Db() {
    if (handle && close) close(handle);
    if (lib) dlclose(lib);
  }

  void open_file(const std::string& path) {
    if (open(path.c_str(), &handle) != kSqliteOk) throw std::runtime_error("failed to open sqlite db: " + path);
    run("CREATE TABLE IF NOT EXISTS sessions ("
        "session_id TEXT PRIMARY KEY,"
        "batch_size INTEGER NOT NULL,"
        "shift_blob BLOB NOT NULL,"
        "wkv_blob BLOB NOT NULL,"
        "wkv32 INTEGER NOT NULL DEFAULT 0,"
        "elapsed_blob BLOB NOT NULL,"
        "last_updated REAL NOT NULL"
        ")",
        "failed to initialize sqlite schema: ", nullptr);
    // databases written before the wkv32 column existed gain it here
    run("ALTER TABLE sessions ADD COLUMN wkv32 INTEGER NOT NULL DEFAULT 0", "failed to migrate sqlite schema: ",
        "duplicate column name");
  }

  void run(const char* sql, const char* what, const char* tolerated) {
    char* err = nullptr;
    if (exec(handle, sql, nullptr, nullptr, &err) == kSqliteOk) return;
    const std::string msg = err ? err : "unknown sqlite error";
    if (err) free_(err);
    if (tolerated && msg.find(tolerated) != std::string::npos) return;
    throw std::runtime_error(what + msg);
  }

  // prepared statement, finalized on scope exit
  struct Stmt {
    Db& db;
    void* s = nullptr;
    Stmt(Db& d, const char* sql) : db(d) { db.prepare(db.handle, sql, -1, &s, nullptr); }
    ~Stmt() { if (s) db.finalize(s); }
  };
};

StateCacheManager& StateCacheManager::instance() {
  static StateCacheManager manager;
  return manager;
}

bool StateCacheManager::database_available() const {
  std::lock_guard<std::mutex> lock(mutex_);
  return db_ != nullptr && db_->handle != nullptr;
}

void StateCacheManager::initialize(int l1_capacity, int l2_capacity, const std::string& db_path) {
  std::lock_guard<std::mutex> lock(mutex_);
  if (initialized_) return;
  l1_capacity_ = l1_capacity;
  l2_capacity_ = l2_capacity;
  db_path_ = db_path;
  db_ = Db::load();
  if (db_) db_->open_file(db_path_);
  initialized_ = true;
}

void StateCacheManager::shutdown() {
  std::lock_guard<std::mutex> lock(mutex_);
  if (!initialized_) return;
  for (const auto& kv : l1_cache_) persist_state_locked(kv.first, copy_to_host(*kv.second.state));
  for (const auto& kv : l2_cache_) persist_state_locked(kv.first, kv.second.state);
  l1_cache_.clear();
  l2_cache_.clear();
  l1_order_.clear();
  l2_order_.clear();
  db_.reset();
  initialized_ = false;
}

StateCacheManager::HostState StateCacheManager::copy_to_host(const GenerationState& state) const {
  HostState host;
  host.batch_size = state.batch_size;
  host.wkv32 = state.wkv32;
  host.shift = download<half, uint16_t>(state.shift, "copy shift to host");
  if (state.wkv32) {
    host.wkv_state32 = download<float, float>(state.wkv_state32, "copy wkv32 state to host");
  } else {
    host.wkv_state16 = download<half, uint16_t>(state.wkv_state, "copy wkv state to host");
  }
  host.elapsed = download<int, int>(state.elapsed, "copy elapsed to host");
  return host;
}

GenerationState StateCacheManager::copy_to_device(const HostState& state) const {
  GenerationState device;
  device.batch_size = state.batch_size;
  device.wkv32 = state.wkv32;
  upload(state.shift, device.shift, "copy shift to device");
  if (state.wkv32) {
    upload(state.wkv_state32, device.wkv_state32, "copy wkv32 state to device");
  } else {
    upload(state.wkv_state16, device.wkv_state, "copy wkv state to device");
  }
  upload(state.elapsed, device.elapsed, "copy elapsed to device");
  return device;
}

std::shared_ptr<GenerationState> StateCacheManager::clone_device_state(const GenerationState& state) const {
  auto clone = std::make_shared<GenerationState>();
  clone->batch_size = state.batch_size;
  clone->wkv32 = state.wkv32;
  duplicate(state.shift, clone->shift, "clone shift");
  if (state.wkv32) {
    duplicate(state.wkv_state32, clone->wkv_state32, "clone wkv32");
  } else {
    duplicate(state.wkv_state, clone->wkv_state, "clone wkv");
  }
  duplicate(state.elapsed, clone->elapsed, "clone elapsed");
  return clone;
}

// Makes `key` the most recently used entry of level 1, then restores the capacities.
void StateCacheManager::insert_l1_locked(const std::string& key, std::shared_ptr<GenerationState> state) {
  l1_order_.push_back(key);
  l1_cache_[key] = L1Entry{std::move(state), std::prev(l1_order_.end())};
  spill_locked();
}

// Least recently used entries move down one level while a level is over capacity: device clone -> host copy
// -> database row (dropped if there is no database).
void StateCacheManager::spill_locked() {
  while (static_cast<int>(l1_cache_.size()) > l1_capacity_) {
    const std::string victim = l1_order_.front();
    auto it = l1_cache_.find(victim);
    HostState host = copy_to_host(*it->second.state);
    l1_order_.pop_front();
    l1_cache_.erase(it);
    l2_order_.push_back(victim);
    l2_cache_[victim] = L2Entry{std::move(host), std::prev(l2_order_.end())};
  }
  while (static_cast<int>(l2_cache_.size()) > l2_capacity_) {
    const std::string victim = l2_order_.front();
    auto it = l2_cache_.find(victim);
    persist_state_locked(victim, it->second.state);
    l2_order_.pop_front();
    l2_cache_.erase(it);
  }
}

void StateCacheManager::persist_state_locked(const std::string& session_id, const HostState& state) {
  if (!db_) return;
  Db::Stmt st(*db_,
              "INSERT OR REPLACE INTO sessions "
              "(session_id, batch_size, shift_blob, wkv_blob, wkv32, elapsed_blob, last_updated) "
              "VALUES (?, ?, ?, ?, ?, ?, ?)");
  if (!st.s) return;
  db_->bind_text(st.s, 1, session_id.c_str(), -1, kTransient);
  db_->bind_int(st.s, 2, state.batch_size);
  db_->bind_blob(st.s, 3, state.shift.data(), static_cast<int>(state.shift.size() * sizeof(uint16_t)), kTransient);
  if (state.wkv32) {
    db_->bind_blob(st.s, 4, state.wkv_state32.data(), static_cast<int>(state.wkv_state32.size() * sizeof(float)),
                   kTransient);
  } else {
    db_->bind_blob(st.s, 4, state.wkv_state16.data(),
                   static_cast<int>(state.wkv_state16.size() * sizeof(uint16_t)), kTransient);
  }
  db_->bind_int(st.s, 5, state.wkv32 ? 1 : 0);
  db_->bind_blob(st.s, 6, state.elapsed.data(), static_cast<int>(state.elapsed.size() * sizeof(int)), kTransient);
  db_->bind_double(st.s, 7, static_cast<double>(std::time(nullptr)));
  db_->step(st.s);
}

std::optional<StateCacheManager::HostState> StateCacheManager::load_state_locked(const std::string& session_id) {
  if (!db_) return std::nullopt;
  Db::Stmt st(*db_, "SELECT batch_size, shift_blob, wkv_blob, wkv32, elapsed_blob FROM sessions WHERE session_id = ?");
  if (!st.s) return std::nullopt;
  db_->bind_text(st.s, 1, session_id.c_str(), -1, kTransient);
  if (db_->step(st.s) != kSqliteRow) return std::nullopt;
  HostState state;
  state.batch_size = db_->column_int(st.s, 0);
  state.wkv32 = db_->column_int(st.s, 3) != 0;
  auto take = [&](int col, auto& vec) {
    using E = typename std::remove_reference_t<decltype(vec)>::value_type;
    const auto* p = static_cast<const E*>(db_->column_blob(st.s, col));
    const int bytes = db_->column_bytes(st.s, col);
    if (p && bytes > 0) vec.assign(p, p + bytes / static_cast<int>(sizeof(E)));
  };
  take(1, state.shift);
  if (state.wkv32) {
    take(2, state.wkv_state32);
  } else {
    take(2, state.wkv_state16);
  }
  take(4, state.elapsed);
  return state;
}

void StateCacheManager::put_state(const std::string& session_id, const GenerationState& state) {
  std::lock_guard<std::mutex> lock(mutex_);
  if (!initialized_ || session_id.empty()) return;
  if (auto it = l1_cache_.find(session_id); it != l1_cache_.end()) {
    l1_order_.erase(it->second.it);
    l1_cache_.erase(it);
  }
  if (auto it = l2_cache_.find(session_id); it != l2_cache_.end()) {
    l2_order_.erase(it->second.it);
    l2_cache_.erase(it);
  }
  insert_l1_locked(session_id, clone_device_state(state));
}

std::optional<GenerationState> StateCacheManager::get_state(const std::string& session_id) {
  std::lock_guard<std::mutex> lock(mutex_);
  if (!initialized_ || session_id.empty()) return std::nullopt;

  if (auto it = l1_cache_.find(session_id); it != l1_cache_.end()) {
    l1_order_.splice(l1_order_.end(), l1_order_, it->second.it);  // now most recently used
    auto copy = clone_device_state(*it->second.state);
    return GenerationState(std::move(*copy));
  }
  if (auto it = l2_cache_.find(session_id); it != l2_cache_.end()) {
    GenerationState device = copy_to_device(it->second.state);
    l2_order_.erase(it->second.it);
    l2_cache_.erase(it);
    insert_l1_locked(session_id, clone_device_state(device));
    return device;
  }
  if (auto host = load_state_locked(session_id); host.has_value()) {
    GenerationState device = copy_to_device(*host);
    insert_l1_locked(session_id, clone_device_state(device));
    return device;
  }
  return std::nullopt;
}

bool StateCacheManager::delete_state_from_any_level(const std::string& session_id) {
  std::lock_guard<std::mutex> lock(mutex_);
  bool found = false;
  if (auto it = l1_cache_.find(session_id); it != l1_cache_.end()) {
    l1_order_.erase(it->second.it);
    l1_cache_.erase(it);
    found = true;
  }
  if (auto it = l2_cache_.find(session_id); it != l2_cache_.end()) {
    l2_order_.erase(it->second.it);
    l2_cache_.erase(it);
    found = true;
  }
  if (db_) {
    Db::Stmt st(*db_, "DELETE FROM sessions WHERE session_id = ?");
    if (st.s) {
      db_->bind_text(st.s, 1, session_id.c_str(), -1, kTransient);
      if (db_->step(st.s) == kSqliteDone && db_->changes(db_->handle) > 0) found = true;
    }
  }
  return found;
}

StateCacheManager::StateSummary StateCacheManager::list_all_states() {
  std::lock_guard<std::mutex> lock(mutex_);
  StateSummary summary;
  for (const auto& kv : l1_cache_) summary.l1_cache.push_back(kv.first);
  for (const auto& kv : l2_cache_) summary.l2_cache.push_back(kv.first);
  if (db_) {
    Db::Stmt st(*db_, "SELECT session_id FROM sessions ORDER BY last_updated DESC");
    while (st.s && db_->step(st.s) == kSqliteRow) {
      const auto* text = reinterpret_cast<const char*>(db_->column_text(st.s, 0));
      if (text) summary.database.emplace_back(text);
    }
  }
  return summary;
}

std::optional<double> StateCacheManager::get_db_timestamp(const std::string& session_id) {
  std::lock_guard<std::mutex> lock(mutex_);
  if (!db_) return std::nullopt;
  Db::Stmt st(*db_, "SELECT last_updated FROM sessions WHERE session_id = ?");
  if (!st.s) return std::nullopt;
  db_->bind_text(st.s, 1, session_id.c_str(), -1, kTransient);
  if (db_->step(st.s) == kSqliteRow) return db_->column_double(st.s, 0);
  return std::nullopt;
}

}  // namespace rwkv7_server
