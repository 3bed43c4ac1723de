// Registries, dialect preference and dispatch of the op layer (see op.h).
#include <algorithm>
#include <mutex>
#include <sstream>

#include "op.h"

namespace raf {
namespace op {

namespace {

template <typename T>
struct Registry {
  std::mutex mu;
  std::map<std::string, std::unique_ptr<T>> entries;
  std::vector<std::string> order;

  T& RegisterOrGet(const std::string& key) {
    std::lock_guard<std::mutex> lock(mu);
    auto it = entries.find(key);
    if (it == entries.end()) {
      it = entries.emplace(key, std::unique_ptr<T>(new T())).first;
      order.push_back(key);
    }
    return *it->second;
  }
  const T* Find(const std::string& key) {
    std::lock_guard<std::mutex> lock(mu);
    auto it = entries.find(key);
    return it == entries.end() ? nullptr : it->second.get();
  }
};

// function-local statics: usable from the static initialisers of other translation units
Registry<OpEnvMaker>& Makers() {
  static Registry<OpEnvMaker> r;
  return r;
}
Registry<Dialect>& Dialects() {
  static Registry<Dialect> r;
  return r;
}
Registry<OpDialect>& OpDialects() {
  static Registry<OpDialect> r;
  return r;
}
struct DeclareEntry {
  FRAFDeclare f;
};
Registry<DeclareEntry>& Declares() {
  static Registry<DeclareEntry> r;
  return r;
}

thread_local std::vector<DialectPreference> g_pref_stack;

std::mutex g_stream_mu;
std::map<int, void*> g_streams;

}  // namespace

// ---- OpEnv ---------------------------------------------------------------------------------
void OpEnv::SetStreamForAllBackends(int device_id, void* stream) {
  std::lock_guard<std::mutex> lock(g_stream_mu);
  g_streams[device_id] = stream;
}
void* OpEnv::GetStream(int device_id) {
  std::lock_guard<std::mutex> lock(g_stream_mu);
  auto it = g_streams.find(device_id);
  return it == g_streams.end() ? nullptr : it->second;
}

// ---- OpEnvMaker ------------------------------------------------------------------------------
OpEnvMaker& OpEnvMaker::RegisterOrGet(const std::string& op_name) { return Makers().RegisterOrGet(op_name); }
const OpEnvMaker* OpEnvMaker::Get(const std::string& op_name) { return Makers().Find(op_name); }
OpEnvPtr OpEnvMaker::Make(const std::string& op_name, const CallValues& call) {
  auto maker = OpEnvMaker::Get(op_name);
  RAF_CHECK(maker != nullptr, "Cannot find an OpEnvMaker registered to " + op_name);
  return OpEnvPtr((*maker)(call));
}

// ---- Dialect ---------------------------------------------------------------------------------
bool Dialect::is_enabled(const std::string& device_type) const {
  return std::find(enable_devices_.begin(), enable_devices_.end(), device_type) != enable_devices_.end();
}
Dialect& Dialect::RegisterOrGet(const std::string& n) { return Dialects().RegisterOrGet(n); }
const Dialect* Dialect::Get(const std::string& n) { return Dialects().Find(n); }
bool Dialect::IsEnabled(const std::string& dialect, const std::string& device_type) {
  const Dialect* d = Get(dialect);
  RAF_CHECK(d != nullptr, "Dialect " + dialect + " is not registered.");
  return d->is_enabled(device_type);
}
std::vector<std::string> Dialect::GetEnabledDialects(const std::string& device_type) {
  std::vector<std::string> ret;
  auto& reg = Dialects();
  std::lock_guard<std::mutex> lock(reg.mu);
  for (const auto& key : reg.order)
    if (reg.entries[key]->is_enabled(device_type)) ret.push_back(key);
  return ret;
}

// ---- OpDialect -------------------------------------------------------------------------------
OpDialect& OpDialect::add_dialect(const std::string& dialect, const std::string& dialect_op, int plevel) {
  for (const auto& e : entries_) {
    RAF_CHECK(e.dialect != dialect, "base operator " + name + " already has a registration on dialect " + dialect);
    RAF_CHECK(e.plevel != plevel, "base operator " + name + " already has a registration with the same plevel");
  }
  auto it = entries_.begin();
  while (it != entries_.end() && it->plevel >= plevel) ++it;
  entries_.insert(it, DialectOpEntry{dialect, dialect_op, plevel});
  return *this;
}
OpDialect& OpDialect::RegisterOrGet(const std::string& base_op) { return OpDialects().RegisterOrGet(base_op); }
const OpDialect* OpDialect::Get(const std::string& base_op) { return OpDialects().Find(base_op); }

std::vector<OpDialect::DialectOpEntry> OpDialect::GetDispatchList(const std::string& base_op,
                                                                  const std::string& device_type) {
  std::vector<DialectOpEntry> enabled;
  const OpDialect* od = Get(base_op);
  if (od == nullptr) return enabled;
  for (const auto& e : od->entries_) {
    const Dialect* d = Dialect::Get(e.dialect);
    RAF_CHECK(d != nullptr, "Dialect " + e.dialect + " is not registered.");
    if (d->is_enabled(device_type)) enabled.push_back(e);
  }
  const DialectPreference* pref = DialectPreference::Current();
  if (pref == nullptr) return enabled;
  std::vector<DialectOpEntry> preferred;
  for (const auto& want : pref->dialects())
    for (const auto& e : enabled)
      if (e.dialect == want) {
        preferred.push_back(e);
        break;
      }
  return preferred;
}

// ---- OpDeclare -------------------------------------------------------------------------------
void OpDeclare::Register(const std::string& base_op, FRAFDeclare f) { Declares().RegisterOrGet(base_op).f = std::move(f); }
const FRAFDeclare* OpDeclare::Get(const std::string& base_op) {
  const DeclareEntry* e = Declares().Find(base_op);
  return e ? &e->f : nullptr;
}

// ---- DialectPreference -------------------------------------------------------------------------
void DialectPreference::EnterWithScope() { g_pref_stack.push_back(*this); }
void DialectPreference::ExitWithScope() {
  RAF_CHECK(!g_pref_stack.empty(), "dialect preference stack is empty");
  g_pref_stack.pop_back();
}
const DialectPreference* DialectPreference::Current() { return g_pref_stack.empty() ? nullptr : &g_pref_stack.back(); }

// ---- Declare + Dispatch --------------------------------------------------------------------------
void RunDeclare(CallValues& call) {
  const FRAFDeclare* f = OpDeclare::Get(call.op_name);
  RAF_CHECK(f != nullptr && *f, "no FRAFDeclare registered for " + call.op_name);
  (*f)(call);
}

OpEnvPtr Dispatch(const CallValues& call) {
  // try the op's own maker first (a dialect op name may be called directly)
  if (const OpEnvMaker* maker = OpEnvMaker::Get(call.op_name)) {
    OpEnvPtr env((*maker)(call));
    if (env != nullptr) return env;
  }
  std::ostringstream tried;
  for (const auto& entry : OpDialect::GetDispatchList(call.op_name, "hip")) {
    if (entry.plevel <= 0) continue;
    tried << " " << entry.dialect_op;
    if (OpEnvPtr env = OpEnvMaker::Make(entry.dialect_op, call)) return env;  // nullptr = declined
  }
  throw Error("Cannot find a valid dispatch for op " + call.op_name + " (tried:" + tried.str() + ")");
}

std::vector<std::string> ListRegisteredOps() {
  auto& reg = OpDialects();
  std::lock_guard<std::mutex> lock(reg.mu);
  return reg.order;
}

}  // namespace op
}  // namespace raf
