// The list of the kernel instances compiled into this library and of those launched so far
// (see instances.h).  Host code only.
#include "instances.h"

#include <stdio.h>
#include <string.h>

#include <mutex>
#include <string>
#include <vector>

#include "api.h"

namespace {

const char* const KIND_NAMES[INST_KINDS] = {"gemm_fma", "gemm_tile", "gemm_stream", "gemm_normed", "gemm_rows",
                                            "gemm_split_reduce", "attention_rows", "attention_prefill",
                                            "attention_decode", "rmsnorm"};

struct Registry {
  std::mutex lock;
  std::vector<std::string> names;
  std::vector<char> hit;
};

// made at first use: instances register themselves while the library's objects are initialised,
// in no order that could be relied on
Registry& registry() {
  static Registry* r = new Registry();
  return *r;
}

}  // namespace

int axk_register_instance(int kind, std::initializer_list<int> params) {
  std::string name = kind >= 0 && kind < INST_KINDS ? KIND_NAMES[kind] : "unknown";
  char sep = '<';
  for (int p : params) {
    name += sep;
    name += std::to_string(p);
    sep = ',';
  }
  if (sep == ',') name += '>';
  Registry& r = registry();
  std::lock_guard<std::mutex> guard(r.lock);
  for (size_t i = 0; i < r.names.size(); ++i)
    if (r.names[i] == name) return (int)i;
  r.names.push_back(name);
  r.hit.push_back(0);
  return (int)r.names.size() - 1;
}

void axk_note_instance(int id) {
  Registry& r = registry();
  if (id >= 0 && id < (int)r.hit.size()) r.hit[id] = 1;
}

// The names, one a line, of every instance (only_hit 0) or of those launched since the last
// reset (only_hit 1) into buf; returns the bytes the whole list needs (with its final zero).
extern "C" long axk_instances(char* buf, long size, int only_hit) {
  Registry& r = registry();
  std::lock_guard<std::mutex> guard(r.lock);
  std::string all;
  for (size_t i = 0; i < r.names.size(); ++i)
    if (!only_hit || r.hit[i]) all += r.names[i] + "\n";
  if (buf != nullptr && size > 0) {
    const size_t n = all.size() < (size_t)size - 1 ? all.size() : (size_t)size - 1;
    memcpy(buf, all.data(), n);
    buf[n] = 0;
  }
  return (long)all.size() + 1;
}

extern "C" void axk_instances_reset(void) {
  Registry& r = registry();
  std::lock_guard<std::mutex> guard(r.lock);
  for (char& h : r.hit) h = 0;
}
