#include "schedule.h"

#include <cmath>
#include <fstream>
#include <sstream>
#include <stdexcept>

namespace engine_c {

namespace {
[[noreturn]] void bad(const std::string &what) { throw std::runtime_error("schedule: " + what); }

bool known_buffer(const std::string &b) { return b == "in" || b == "out" || b == "ws"; }
}  // namespace

int Schedule::elemBytes() const {
  if (dtype == "f64") return 8;
  if (dtype == "f32" || dtype == "i32" || dtype == "u32") return 4;
  if (dtype == "bf16" || dtype == "f16") return 2;
  if (dtype == "f8e4m3" || dtype == "f8e5m2") return 1;
  bad("unknown dtype '" + dtype + "'");
}

void Schedule::validate() const {
  (void)elemBytes();
  if (compute != "sum" && compute != "prod" && compute != "min" && compute != "max")
    bad("unknown compute '" + compute + "'");
  if (devices < 1) bad("devices must be >= 1");
  if (elems_per_device < 0) bad("elems_per_device must be >= 0");
  const int n = (int)ops.size();
  for (int i = 0; i < n; ++i) {
    const ScheduleOp &o = ops[i];
    const std::string at = "op " + std::to_string(i) + ": ";
    if (o.count < 0) bad(at + "negative count");
    if (o.isSignal()) {
      if (o.slot < 0 || o.slot >= 256) bad(at + "signal slot outside [0, 256)");
      if (o.parts < 1 || o.slot + o.parts > 256) bad(at + "a signal of " + std::to_string(o.parts) + " words does not fit the 256 slots");
      if (o.count > 0xffff) bad(at + "signal value outside [0, 65535]");
      if (!o.srcs.empty() || !o.dsts.empty()) bad(at + "a signal op has no data operands");
      if (o.deps.size() > 255) bad(at + "more than 255 dependencies");
      for (int d : o.deps)
        if (d < 0 || d >= n || d == i) bad(at + "dependency " + std::to_string(d) + " is not another op");
      continue;
    }
    if ((o.kind == ScheduleOp::REDUCE) != o.reduce) bad(at + "kind and reduce flag disagree");
    if (o.srcs.empty() || o.srcs.size() > 8) bad(at + "needs 1..8 sources");
    if (o.dsts.empty() || o.dsts.size() > 8) bad(at + "needs 1..8 destinations");
    if (o.srcs.size() + o.dsts.size() > 10) bad(at + "more than 10 operands in all");
    if (!o.reduce && o.srcs.size() != 1) bad(at + "COPY takes exactly one source");
    for (const auto *list : {&o.srcs, &o.dsts})
      for (const ScheduleOperand &x : *list) {
        if (!known_buffer(x.buffer)) bad(at + "unknown buffer '" + x.buffer + "'");
        if (x.device < 0 || x.device >= devices) bad(at + "device outside [0, devices)");
        if (x.offset < 0) bad(at + "negative offset");
        if (x.buffer != "ws" && x.offset + o.count > elems_per_device)
          bad(at + "operand runs past elems_per_device");
      }
    for (const ScheduleOperand &x : o.dsts)
      if (x.buffer == "in") bad(at + "the input tensor is read-only");
    if (o.deps.size() > 255) bad(at + "more than 255 dependencies");
    for (int d : o.deps)
      if (d < 0 || d >= n || d == i) bad(at + "dependency " + std::to_string(d) + " is not another op");
  }
  (void)topologicalOrder();  // throws on a cycle
}

std::vector<int> Schedule::topologicalOrder() const {
  const int n = (int)ops.size();
  // successor lists in edge-insertion order: for op 0, 1, ... one edge per dependency
  std::vector<std::vector<int>> succ(n);
  for (int i = 0; i < n; ++i)
    for (int d : ops[i].deps) {
      if (d < 0 || d >= n) bad("dependency outside the op list");
      succ[d].push_back(i);
    }
  std::vector<char> state(n, 0);
  std::vector<int> post;
  post.reserve(n);
  std::vector<std::pair<int, size_t>> stack;
  for (int root = 0; root < n; ++root) {
    if (state[root]) continue;
    stack.push_back({root, 0});
    state[root] = 1;
    while (!stack.empty()) {
      auto &[v, i] = stack.back();
      if (i < succ[v].size()) {
        const int w = succ[v][i++];
        if (state[w] == 1) bad("dependency graph has a cycle");
        if (state[w] == 0) {
          state[w] = 1;
          stack.push_back({w, 0});
        }
      } else {
        state[v] = 2;
        post.push_back(v);
        stack.pop_back();
      }
    }
  }
  return std::vector<int>(post.rbegin(), post.rend());
}

std::string Schedule::serialize() const {
  std::ostringstream os;
  // version 2 where a signal has a word per part (the only thing version 1 cannot say)
  bool by_part = false;
  for (const ScheduleOp &o : ops) by_part = by_part || (o.isSignal() && o.parts > 1);
  os << "pccl-schedule " << (by_part ? 2 : 1) << "\n";
  os << "name " << (name.empty() ? "unnamed" : name) << "\n";
  os << "dtype " << dtype << "\ncompute " << compute << "\n";
  os << "devices " << devices << "\nelems_per_device " << elems_per_device << "\n";
  os << "ops " << ops.size() << "\n";
  for (size_t i = 0; i < ops.size(); ++i) {
    const ScheduleOp &o = ops[i];
    static const char *kinds[] = {"COPY", "REDUCE", "NOTIFY", "GET_NOTIFIED"};
    os << "op " << i << ' ' << kinds[o.kind] << ' ' << o.count << " deps " << o.deps.size();
    for (int d : o.deps) os << ' ' << d;
    if (o.isSignal()) {
      os << " slot " << o.slot;
      if (by_part) os << " parts " << o.parts;
      os << "\n";
      continue;
    }
    os << " src " << o.srcs.size();
    for (const auto &x : o.srcs) os << ' ' << x.buffer << ' ' << x.device << ' ' << x.offset;
    os << " dst " << o.dsts.size();
    for (const auto &x : o.dsts) os << ' ' << x.buffer << ' ' << x.device << ' ' << x.offset;
    os << "\n";
  }
  return os.str();
}

Schedule Schedule::parse(const std::string &text) {
  // strip comment lines, then read one token stream
  std::istringstream lines(text);
  std::string line, body;
  while (std::getline(lines, line)) {
    const size_t p = line.find_first_not_of(" \t\r");
    if (p == std::string::npos || line[p] == '#') continue;
    body += line;
    body += '\n';
  }
  std::istringstream in(body);
  auto word = [&](const char *what) {
    std::string w;
    if (!(in >> w)) bad(std::string("unexpected end of file, expected ") + what);
    return w;
  };
  auto expect = [&](const char *kw) {
    const std::string w = word(kw);
    if (w != kw) bad(std::string("expected '") + kw + "', found '" + w + "'");
  };
  auto integer = [&](const char *what) {
    const std::string w = word(what);
    size_t used = 0;
    long v = 0;
    try {
      v = std::stol(w, &used);
    } catch (const std::exception &) {
      used = 0;
    }
    if (used != w.size()) bad(std::string("expected an integer for ") + what + ", found '" + w + "'");
    return v;
  };
  Schedule s;
  expect("pccl-schedule");
  const long version = integer("version");
  if (version != 1 && version != 2) bad("unsupported format version " + std::to_string(version));
  expect("name");
  s.name = word("name");
  expect("dtype");
  s.dtype = word("dtype");
  expect("compute");
  s.compute = word("compute");
  expect("devices");
  s.devices = (int)integer("devices");
  expect("elems_per_device");
  s.elems_per_device = integer("elems_per_device");
  expect("ops");
  const long n = integer("op count");
  if (n < 0 || n > (1l << 24)) bad("op count out of range");
  s.ops.resize((size_t)n);
  for (long i = 0; i < n; ++i) {
    expect("op");
    if (integer("op id") != i) bad("op ids must be 0, 1, 2, ... in file order");
    ScheduleOp &o = s.ops[(size_t)i];
    const std::string kind = word("op kind");
    if (kind == "REDUCE") o.kind = ScheduleOp::REDUCE;
    else if (kind == "COPY") o.kind = ScheduleOp::COPY;
    else if (kind == "NOTIFY") o.kind = ScheduleOp::NOTIFY;
    else if (kind == "GET_NOTIFIED") o.kind = ScheduleOp::GET_NOTIFIED;
    else bad("op " + std::to_string(i) + ": unknown kind '" + kind + "'");
    o.reduce = o.kind == ScheduleOp::REDUCE;
    o.count = integer("count");
    expect("deps");
    const long nd = integer("dependency count");
    if (nd < 0 || nd > 255) bad("op " + std::to_string(i) + ": dependency count out of range");
    for (long d = 0; d < nd; ++d) o.deps.push_back((int)integer("dependency"));
    if (o.isSignal()) {
      expect("slot");
      o.slot = (int)integer("slot");
      if (version >= 2) {
        expect("parts");
        const long k = integer("parts");
        if (k < 1 || k > 256) bad("op " + std::to_string(i) + ": parts out of range");
        o.parts = (int)k;
      }
      continue;
    }
    for (int side = 0; side < 2; ++side) {
      expect(side == 0 ? "src" : "dst");
      const long k = integer("operand count");
      if (k < 0 || k > 8) bad("op " + std::to_string(i) + ": operand count out of range");
      for (long j = 0; j < k; ++j) {
        ScheduleOperand x;
        x.buffer = word("buffer");
        x.device = (int)integer("device");
        x.offset = integer("offset");
        (side == 0 ? o.srcs : o.dsts).push_back(x);
      }
    }
  }
  std::string extra;
  if (in >> extra) bad("trailing text after the last op: '" + extra + "'");
  s.validate();
  return s;
}

Schedule Schedule::load(const std::string &path) {
  std::ifstream f(path, std::ios::binary);
  if (!f.is_open()) throw std::runtime_error("Failed to open file: " + path);
  std::ostringstream ss;
  ss << f.rdbuf();
  return parse(ss.str());
}

void Schedule::save(const std::string &path) const {
  std::ofstream f(path, std::ios::binary | std::ios::trunc);
  if (!f.is_open()) throw std::runtime_error("Failed to open file for writing: " + path);
  f << serialize();
  if (!f.good()) throw std::runtime_error("Failed to write file: " + path);
}

long appendRingAllReduce(Schedule &s, long chunk_elems, long base) {
  const int W = s.devices;
  std::vector<int> prev(W, -1), cur(W, -1);
  auto mod = [W](int x) { return ((x % W) + W) % W; };
  for (int step = 1; step < W; ++step) {  // reduce-scatter
    for (int r = 0; r < W; ++r) {
      const int c = mod(r - step), p = mod(r - 1);
      const long off = base + (long)c * chunk_elems;
      ScheduleOp o;
      o.kind = ScheduleOp::REDUCE;
      o.reduce = true;
      o.count = chunk_elems;
      o.srcs.push_back({step == 1 ? "in" : "out", p, off});  // partial sum arriving from rank r-1
      o.srcs.push_back({"in", r, off});                      // own contribution
      o.dsts.push_back({"out", r, off});
      if (step > 1) o.deps.push_back(prev[p]);
      cur[r] = (int)s.ops.size();
      s.ops.push_back(std::move(o));
    }
    prev = cur;
  }
  for (int step = 1; step < W; ++step) {  // all-gather
    for (int r = 0; r < W; ++r) {
      const int c = mod(r - step + 1), p = mod(r - 1);
      const long off = base + (long)c * chunk_elems;
      ScheduleOp o;
      o.reduce = false;
      o.count = chunk_elems;
      o.srcs.push_back({"out", p, off});
      o.dsts.push_back({"out", r, off});
      o.deps.push_back(prev[p]);
      cur[r] = (int)s.ops.size();
      s.ops.push_back(std::move(o));
    }
    prev = cur;
  }
  const long end = base + (long)W * chunk_elems;
  if (end > s.elems_per_device) s.elems_per_device = end;
  return end;
}

long appendRingReduceScatter(Schedule &s, long chunk_elems, long base) {
  const int W = s.devices;
  std::vector<int> prev(W, -1), cur(W, -1);
  auto mod = [W](int x) { return ((x % W) + W) % W; };
  for (int step = 1; step < W; ++step) {
    for (int r = 0; r < W; ++r) {
      const int c = mod(r - step), p = mod(r - 1);
      const long off = base + (long)c * chunk_elems;
      ScheduleOp o;
      o.kind = ScheduleOp::REDUCE;
      o.reduce = true;
      o.count = chunk_elems;
      o.srcs.push_back({step == 1 ? "in" : "out", p, off});
      o.srcs.push_back({"in", r, off});
      o.dsts.push_back({"out", r, off});
      if (step > 1) o.deps.push_back(prev[p]);
      cur[r] = (int)s.ops.size();
      s.ops.push_back(std::move(o));
    }
    prev = cur;
  }
  const long end = base + (long)W * chunk_elems;
  if (end > s.elems_per_device) s.elems_per_device = end;
  return end;
}

long appendRingAllGather(Schedule &s, long chunk_elems, long base) {
  const int W = s.devices;
  std::vector<int> prev(W, -1), cur(W, -1);
  auto mod = [W](int x) { return ((x % W) + W) % W; };
  for (int r = 0; r < W; ++r) {  // own chunk: in -> out
    ScheduleOp o;
    o.count = chunk_elems;
    o.srcs.push_back({"in", r, base + (long)r * chunk_elems});
    o.dsts.push_back({"out", r, base + (long)r * chunk_elems});
    prev[r] = (int)s.ops.size();
    s.ops.push_back(std::move(o));
  }
  for (int step = 1; step < W; ++step) {
    for (int r = 0; r < W; ++r) {
      const int c = mod(r - step), p = mod(r - 1);
      const long off = base + (long)c * chunk_elems;
      ScheduleOp o;
      o.count = chunk_elems;
      o.srcs.push_back({"out", p, off});
      o.dsts.push_back({"out", r, off});
      o.deps.push_back(prev[p]);
      cur[r] = (int)s.ops.size();
      s.ops.push_back(std::move(o));
    }
    prev = cur;
  }
  const long end = base + (long)W * chunk_elems;
  if (end > s.elems_per_device) s.elems_per_device = end;
  return end;
}

long appendBroadcast(Schedule &s, long elems, int root, long base) {
  const int W = s.devices;
  if (W > 8) bad("broadcast names one destination per device: at most 8 devices");
  if (root < 0 || root >= W) bad("broadcast root outside the devices");
  ScheduleOp o;
  o.count = elems;
  o.srcs.push_back({"in", root, base});
  o.dsts.push_back({"out", root, base});
  for (int r = 0; r < W; ++r)
    if (r != root) o.dsts.push_back({"out", r, base});
  s.ops.push_back(std::move(o));
  const long end = base + elems;
  if (end > s.elems_per_device) s.elems_per_device = end;
  return end;
}

long appendAllToAll(Schedule &s, long chunk_elems, long base) {
  const int W = s.devices;
  for (int r = 0; r < W; ++r)
    for (int d = 0; d < W; ++d) {
      ScheduleOp o;
      o.count = chunk_elems;
      o.srcs.push_back({"in", r, base + (long)d * chunk_elems});
      o.dsts.push_back({"out", d, base + (long)r * chunk_elems});
      s.ops.push_back(std::move(o));
    }
  const long end = base + (long)W * chunk_elems;
  if (end > s.elems_per_device) s.elems_per_device = end;
  return end;
}

long appendDirectAllReduce(Schedule &s, long slice_elems, long base) {
  const int W = s.devices;
  if (W > 8) bad("direct all-reduce supports at most 8 devices (8 inputs per op)");
  for (int d = 0; d < W; ++d) {
    const long off = base + (long)d * slice_elems;
    ScheduleOp red;
    red.reduce = W > 1;
    red.kind = W > 1 ? ScheduleOp::REDUCE : ScheduleOp::COPY;
    red.count = slice_elems;
    for (int r = 0; r < W; ++r) red.srcs.push_back({"in", r, off});  // fixed order: rank 0 first
    red.dsts.push_back({"out", d, off});
    const int red_id = (int)s.ops.size();
    s.ops.push_back(std::move(red));
    if (W > 1) {  // broadcast store to the other devices
      ScheduleOp bc;
      bc.reduce = false;
      bc.count = slice_elems;
      bc.srcs.push_back({"out", d, off});
      for (int r = 0; r < W; ++r)
        if (r != d) bc.dsts.push_back({"out", r, off});
      bc.deps.push_back(red_id);
      s.ops.push_back(std::move(bc));
    }
  }
  const long end = base + (long)W * slice_elems;
  if (end > s.elems_per_device) s.elems_per_device = end;
  return end;
}

namespace {
unsigned long mix64(unsigned long z) {
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ul;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebul;
  return z ^ (z >> 31);
}
}  // namespace

Schedule makeSmallMessageSchedule(int devices, int n_slices, int n_extra, unsigned long seed,
                                  long lo_bytes, long hi_bytes, const std::string &dtype) {
  Schedule s;
  s.name = "small_message_allreduce";
  s.dtype = dtype;
  s.compute = "sum";
  s.devices = devices;
  const int es = s.elemBytes();
  const unsigned long golden = 0x9e3779b97f4a7c15ul;
  auto size_of = [&](int i) {
    const double u = (double)(mix64(seed * golden + (unsigned long)(i + 1) * golden) >> 11) / 9007199254740992.0;
    const long bytes = (long)((double)lo_bytes * std::exp(u * std::log((double)hi_bytes / (double)lo_bytes)));
    return std::max<long>(1, bytes / es);
  };
  long base = 0;
  for (int k = 0; k < n_slices; ++k) base = appendRingAllReduce(s, size_of(k), base);
  long round_max = 0;
  for (int i = 0; i < n_extra; ++i) {  // independent copies, device i % W, one region per round
    const int r = i % devices;
    const long n = size_of(n_slices + i);
    ScheduleOp o;
    o.count = n;
    o.srcs.push_back({"in", r, base});
    o.dsts.push_back({"out", r, base});
    s.ops.push_back(std::move(o));
    round_max = std::max(round_max, n);
    if (r == devices - 1 || i == n_extra - 1) {
      base += round_max;
      round_max = 0;
    }
  }
  s.elems_per_device = std::max(s.elems_per_device, base);
  s.validate();
  return s;
}

}  // namespace engine_c
