// tq_run: a host in C++ without Python, from a model folder to generated tokens through the step executor.
//
//   tq_run --lib libtq_<type>.so --plan PLAN --model DIR -p "5,17,3;8,1" [-n 8]
//
// In the manner of the reference's command line (/root/reference/tools/quant.c:187-346: load the model, run the
// prompt, then token by token, stop on an end token): reads the model's plan (engine/plan_file.py writes it from the
// architecture's own description: parts, sizes, which tensors make up which parameter), reads model.safetensors by
// tensor name, places the parameters on the GPU, fills the executor's descriptors (host/engine.h), keeps a cache of
// one slot per prompt, runs the prompts as one step and then one token per sequence and step, choosing the most
// likely token each time (tq_argmax), and prints the tokens as `bin/quant -T 0` does.  Greedy only; the prompts are
// token ids.  It exists to show that a host needs nothing of this library but its C entry points.
#include <dlfcn.h>
#include <fcntl.h>
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <fstream>
#include <map>
#include <sstream>
#include <string>
#include <vector>

#include "engine.h"

namespace {

[[noreturn]] void die(const std::string& what) {
  fprintf(stderr, "tq_run: %s\n", what.c_str());
  exit(1);
}

#define HIP_OK(call)                                                                              \
  do {                                                                                            \
    hipError_t e__ = (call);                                                                      \
    if (e__ != hipSuccess) die(std::string(#call) + ": " + hipGetErrorString(e__));               \
  } while (0)

// ------------------------------------------------------------------------------------------ safetensors
struct Tensor {
  std::string dtype;
  std::vector<int64_t> shape;
  size_t begin = 0, end = 0;
};

// The header of a safetensors file is one JSON object of objects; this reads exactly that much JSON.
struct Json {
  const char* p;
  const char* end;
  void blank() {
    while (p < end && (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r')) ++p;
  }
  bool take(char c) {
    blank();
    if (p < end && *p == c) {
      ++p;
      return true;
    }
    return false;
  }
  void need(char c) {
    if (!take(c)) die(std::string("model.safetensors: header is not the JSON expected (wanted '") + c + "')");
  }
  std::string string() {
    need('"');
    std::string s;
    while (p < end && *p != '"') {
      if (*p == '\\' && p + 1 < end) {
        ++p;
        if (*p == 'u') {      // tensor names are ASCII; a \u escape keeps its text
          s += "\\u";
        } else {
          s += *p == 'n' ? '\n' : *p == 't' ? '\t' : *p;
        }
        ++p;
      } else {
        s += *p++;
      }
    }
    need('"');
    return s;
  }
  double number() {
    blank();
    char* stop = nullptr;
    const double v = strtod(p, &stop);
    if (stop == p) die("model.safetensors: a number was expected in the header");
    p = stop;
    return v;
  }
  void skip() {        // any value
    blank();
    if (p >= end) die("model.safetensors: header ends early");
    if (*p == '"') {
      string();
    } else if (*p == '{') {
      ++p;
      if (take('}')) return;
      do {
        string();
        need(':');
        skip();
      } while (take(','));
      need('}');
    } else if (*p == '[') {
      ++p;
      if (take(']')) return;
      do skip();
      while (take(','));
      need(']');
    } else {
      while (p < end && *p != ',' && *p != '}' && *p != ']') ++p;
    }
  }
};

struct Safetensors {
  const unsigned char* data = nullptr;     // behind the header
  size_t bytes = 0;
  std::map<std::string, Tensor> tensors;

  explicit Safetensors(const std::string& path) {
    const int fd = open(path.c_str(), O_RDONLY);
    if (fd < 0) die("cannot open " + path);
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size < 8) die(path + " is no safetensors file");
    void* map = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    if (map == MAP_FAILED) die("cannot map " + path);
    close(fd);
    const unsigned char* base = (const unsigned char*)map;
    uint64_t n = 0;
    memcpy(&n, base, 8);
    if (n > (uint64_t)st.st_size - 8) die(path + ": the header is longer than the file");
    data = base + 8 + n;
    bytes = (size_t)st.st_size - 8 - n;
    Json j{(const char*)base + 8, (const char*)base + 8 + n};
    j.need('{');
    if (!j.take('}')) {
      do {
        const std::string name = j.string();
        j.need(':');
        if (name == "__metadata__") {
          j.skip();
          continue;
        }
        Tensor t;
        j.need('{');
        do {
          const std::string key = j.string();
          j.need(':');
          if (key == "dtype") {
            t.dtype = j.string();
          } else if (key == "shape") {
            j.need('[');
            if (!j.take(']')) {
              do t.shape.push_back((int64_t)j.number());
              while (j.take(','));
              j.need(']');
            }
          } else if (key == "data_offsets") {
            j.need('[');
            t.begin = (size_t)j.number();
            j.need(',');
            t.end = (size_t)j.number();
            j.need(']');
          } else {
            j.skip();
          }
        } while (j.take(','));
        j.need('}');
        if (t.end < t.begin || t.end > bytes) die("tensor " + name + " lies outside the file");
        tensors[name] = t;
      } while (j.take(','));
      j.need('}');
    }
  }
};

// ------------------------------------------------------------------------------------------ number formats
float bf16_to_f32(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
uint16_t f32_to_bf16(float f) {      // round to nearest even; NaN stays NaN
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
float f16_to_f32(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000) << 16, exp = (h >> 10) & 31, man = h & 1023;
  uint32_t u;
  if (exp == 0) {
    if (man == 0) {
      u = sign;
    } else {
      int e = -1;
      uint32_t m = man;
      do {
        ++e;
        m <<= 1;
      } while (!(m & 1024));
      u = sign | ((uint32_t)(127 - 15 - e) << 23) | ((m & 1023) << 13);
    }
  } else if (exp == 31) {
    u = sign | 0x7f800000u | (man << 13);
  } else {
    u = sign | ((exp + 112) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &u, 4);
  return f;
}

// ------------------------------------------------------------------------------------------ the plan
struct Param {
  int layer = 0;
  std::string slot, attr, role, how;
  std::vector<int64_t> shape, splits;
  std::vector<std::string> names;
};
struct PartLine {
  int layer = 0;
  std::string slot, kind;
  std::map<std::string, std::string> args;
  double num(const std::string& key, double otherwise) const {
    auto it = args.find(key);
    return it == args.end() ? otherwise : atof(it->second.c_str());
  }
  double need(const std::string& key) const {
    auto it = args.find(key);
    if (it == args.end()) die("plan: part " + slot + " (" + kind + ") of layer " + std::to_string(layer) + " has no " + key);
    return atof(it->second.c_str());
  }
  std::string text(const std::string& key, const std::string& otherwise) const {
    auto it = args.find(key);
    return it == args.end() ? otherwise : it->second;
  }
};
struct Plan {
  std::string architecture, act;
  std::map<std::string, std::string> model;
  std::vector<int> stop;
  std::vector<Param> params;
  std::vector<PartLine> parts;
  std::map<std::pair<int, std::string>, std::vector<uint32_t>> tables;
  std::vector<std::string> blocks;
  std::vector<std::pair<int, int>> entries;     // layer, cache_of
  bool tied = false;

  const PartLine& part(int layer, const std::string& slot) const {
    for (const PartLine& p : parts)
      if (p.layer == layer && p.slot == slot) return p;
    die("plan: layer " + std::to_string(layer) + " has no part " + slot);
  }
  const Param* param(int layer, const std::string& slot, const std::string& attr) const {
    for (const Param& p : params)
      if (p.layer == layer && p.slot == slot && p.attr == attr) return &p;
    return nullptr;
  }
};

void key_values(std::istringstream& in, std::map<std::string, std::string>& out) {
  std::string word;
  while (in >> word) {
    const size_t eq = word.find('=');
    if (eq == std::string::npos) die("plan: '" + word + "' is no key=value");
    out[word.substr(0, eq)] = word.substr(eq + 1);
  }
}

Plan read_plan(const std::string& path) {
  std::ifstream f(path);
  if (!f) die("cannot open plan " + path);
  Plan plan;
  std::string line;
  if (!std::getline(f, line) || line != "tqplan 1") die(path + " is no plan file of version 1");
  while (std::getline(f, line)) {
    std::istringstream in(line);
    std::string what;
    if (!(in >> what)) continue;
    if (what == "model") {
      in >> plan.architecture;
      key_values(in, plan.model);
      plan.act = plan.model["act"];
    } else if (what == "stop") {
      int n = 0;
      in >> n;
      for (int i = 0, t; i < n && (in >> t); ++i) plan.stop.push_back(t);
    } else if (what == "param") {
      Param p;
      int ndim = 0, n_names = 0;
      in >> p.layer >> p.slot >> p.attr >> p.role >> p.how >> ndim;
      for (int i = 0; i < ndim; ++i) {
        int64_t d;
        in >> d;
        p.shape.push_back(d);
      }
      in >> n_names;
      for (int i = 0; i < n_names; ++i) {
        std::string name;
        in >> name;
        p.names.push_back(name);
      }
      std::string more;
      if (in >> more && more == "splits") {
        int64_t s;
        while (in >> s) p.splits.push_back(s);
      }
      if (!in.eof() && in.fail()) die("plan: cannot read '" + line + "'");
      plan.params.push_back(p);
    } else if (what == "tied") {
      plan.tied = true;
    } else if (what == "layer") {
      int i;
      std::string kind;
      in >> i >> kind;
      if (i != (int)plan.blocks.size()) die("plan: layers are out of order");
      plan.blocks.push_back(kind);
    } else if (what == "part") {
      PartLine p;
      in >> p.layer >> p.slot >> p.kind;
      key_values(in, p.args);
      plan.parts.push_back(p);
    } else if (what == "table") {
      int layer, n;
      std::string slot, name;
      in >> layer >> slot >> name >> n;
      std::vector<uint32_t> bits;
      for (int i = 0; i < n; ++i) {
        std::string hex;
        in >> hex;
        bits.push_back((uint32_t)strtoul(hex.c_str(), nullptr, 16));
      }
      plan.tables[{layer, slot}] = bits;
    } else if (what == "entry") {
      int e;
      std::map<std::string, std::string> kv;
      in >> e;
      key_values(in, kv);
      if (e != (int)plan.entries.size()) die("plan: schedule entries are out of order");
      plan.entries.push_back({atoi(kv["layer"].c_str()), atoi(kv["cache_of"].c_str())});
    } else {
      die("plan: unknown line '" + line + "'");
    }
  }
  return plan;
}

// ------------------------------------------------------------------------------------------ parameters on the device
struct Loader {
  const Safetensors& file;
  bool act_bf16;
  std::vector<std::string> missing, wrong;
  size_t placed = 0;

  // The type a parameter is kept in: as weights/loader.py decides it.
  int kept_type(const Param& p) const {
    if (!act_bf16) return 0;
    bool stored32 = false;
    for (const std::string& n : p.names) {
      auto it = file.tensors.find(n);
      if (it != file.tensors.end() && it->second.dtype == "F32") stored32 = true;
    }
    const bool rounded = p.role == "matrix" || p.role == "table";
    return stored32 && !rounded ? 0 : 1;
  }

  tq_weight place(const Param* p) {
    tq_weight w{nullptr, 0};
    if (!p) return w;
    int64_t total = 1;
    for (int64_t d : p->shape) total *= d;
    const int type = kept_type(*p);
    const size_t esz = type ? 2 : 4;
    std::vector<unsigned char> host((size_t)total * esz);
    int64_t at = 0;
    for (size_t i = 0; i < p->names.size(); ++i) {
      int64_t piece = total;
      if (p->how == "stack") piece = total / p->shape[0];
      if (p->how == "concat") piece = total / p->shape[0] * p->splits[i];
      auto it = file.tensors.find(p->names[i]);
      if (it == file.tensors.end()) {
        missing.push_back(p->names[i]);
        continue;
      }
      const Tensor& t = it->second;
      int64_t have = 1;
      for (int64_t d : t.shape) have *= d;
      const size_t src_esz = t.dtype == "F32" ? 4 : (t.dtype == "BF16" || t.dtype == "F16") ? 2 : 0;
      if (have != piece || src_esz == 0 || t.end - t.begin != (size_t)have * src_esz) {
        wrong.push_back(p->names[i]);
        continue;
      }
      const unsigned char* src = file.data + t.begin;
      for (int64_t j = 0; j < piece; ++j) {
        float v;
        if (t.dtype == "F32") {
          memcpy(&v, src + 4 * j, 4);
        } else {
          uint16_t h;
          memcpy(&h, src + 2 * j, 2);
          v = t.dtype == "BF16" ? bf16_to_f32(h) : f16_to_f32(h);
        }
        if (type) {
          const uint16_t b = f32_to_bf16(v);
          memcpy(&host[(size_t)(at + j) * 2], &b, 2);
        } else {
          memcpy(&host[(size_t)(at + j) * 4], &v, 4);
        }
      }
      at += piece;
    }
    void* dev = nullptr;
    HIP_OK(hipMalloc(&dev, host.size() + 256));
    HIP_OK(hipMemcpy(dev, host.data(), host.size(), hipMemcpyHostToDevice));
    placed += host.size();
    w.ptr = dev;
    w.wtype = type;
    return w;
  }
};

std::vector<std::vector<int>> parse_prompts(const std::string& text) {
  std::vector<std::vector<int>> prompts;
  std::stringstream all(text);
  std::string one;
  while (std::getline(all, one, ';')) {
    std::vector<int> toks;
    std::stringstream s(one);
    std::string t;
    while (std::getline(s, t, ',')) {
      if (t.find_first_not_of(" \t") == std::string::npos) continue;
      toks.push_back(atoi(t.c_str()));
    }
    if (!toks.empty()) prompts.push_back(toks);
  }
  return prompts;
}

int gate_code(const std::string& name) {      // numbered by the lines of gates.def, as the kernels number them
  static const char* const names[] = {
#define TQ_GATE(gate, expr) #gate,
#include "../gates.def"
#undef TQ_GATE
  };
  for (size_t i = 0; i < sizeof(names) / sizeof(names[0]); ++i)
    if (name == names[i]) return (int)i;
  die("plan: unknown activation " + name);
}

}  // namespace

int main(int argc, char** argv) {
  std::string lib_path, plan_path, model_dir, prompt_text = "1";
  int max_new = 8;
  for (int i = 1; i < argc; ++i) {
    const std::string a = argv[i];
    auto value = [&]() -> std::string {
      if (i + 1 >= argc) die("option " + a + " needs a value");
      return argv[++i];
    };
    if (a == "--lib") lib_path = value();
    else if (a == "--plan") plan_path = value();
    else if (a == "--model") model_dir = value();
    else if (a == "-p") prompt_text = value();
    else if (a == "-n") max_new = atoi(value().c_str());
    else die("unknown option " + a + " (usage: tq_run --lib LIB --plan PLAN --model DIR -p \"5,17,3;8,1\" [-n 8])");
  }
  if (lib_path.empty() || plan_path.empty() || model_dir.empty()) die("--lib, --plan and --model are needed");

  // the kernel library: the executor and the choice of the most likely token are all this host calls
  void* lib = dlopen(lib_path.c_str(), RTLD_NOW | RTLD_LOCAL);
  if (!lib) die(std::string("cannot load ") + lib_path + ": " + dlerror());
  auto step_workspace = (decltype(&tq_step_workspace))dlsym(lib, "tq_step_workspace");
  auto step_forward = (decltype(&tq_step_forward))dlsym(lib, "tq_step_forward");
  auto last_error = (decltype(&tq_engine_last_error))dlsym(lib, "tq_engine_last_error");
  typedef int (*argmax_fn)(const float*, int, int, int*, hipStream_t);
  auto argmax = (argmax_fn)dlsym(lib, "tq_argmax");
  if (!step_workspace || !step_forward || !last_error || !argmax) die(lib_path + " holds no step executor");
  const bool lib_bf16 = dlsym(lib, "tq_gemm_mfma") != nullptr;

  const Plan plan = read_plan(plan_path);
  const bool act_bf16 = plan.act == "bfloat16";
  if (act_bf16 != lib_bf16) die("the plan is for " + plan.act + " activations, the library for the other type");
  const int act_bytes = act_bf16 ? 2 : 4;
  auto model_num = [&](const char* key) {
    auto it = plan.model.find(key);
    if (it == plan.model.end()) die(std::string("plan: the model line has no ") + key);
    return atof(it->second.c_str());
  };
  const int64_t V = (int64_t)model_num("vocab"), H = (int64_t)model_num("hidden");
  const int n_layers = (int)model_num("n_layers"), n_entries = (int)model_num("n_entries");
  if ((int)plan.blocks.size() != n_layers || (int)plan.entries.size() != n_entries) die("plan: layers or entries are missing");

  std::vector<std::vector<int>> prompts = parse_prompts(prompt_text);
  if (prompts.empty()) die("no prompt");
  for (auto& p : prompts)
    for (int t : p)
      if (t < 0 || t >= V) die("token " + std::to_string(t) + " is outside the vocabulary of " + std::to_string(V));

  HIP_OK(hipSetDevice(0));
  Safetensors file(model_dir + "/model.safetensors");
  Loader load{file, act_bf16};
  std::vector<tq_layer_desc> layers((size_t)n_layers);
  for (int l = 0; l < n_layers; ++l) {
    if (plan.blocks[l] != "prenorm") die("layer " + std::to_string(l) + ": this host knows the prenorm arrangement only");
    tq_layer_desc& d = layers[l];
    memset(&d, 0, sizeof(d));
    const PartLine &n1 = plan.part(l, "mixer_norm"), &mx = plan.part(l, "mixer"), &n2 = plan.part(l, "ffn_norm"),
                   &ff = plan.part(l, "ffn"), &pos = plan.part(l, "mixer.position");
    if (n1.kind != "rmsnorm" || n2.kind != "rmsnorm" || mx.kind != "gqa_attention")
      die("layer " + std::to_string(l) + ": this host knows rmsnorm and gqa_attention");
    if (mx.args.count("qk_norm_eps")) die("layer " + std::to_string(l) + ": a norm of the heads is not known to the executor");
    d.mixer_norm = {load.place(plan.param(l, "mixer_norm", "weight")), n1.need("eps")};
    d.ffn_norm = {load.place(plan.param(l, "ffn_norm", "weight")), n2.need("eps")};
    tq_attention_desc& a = d.attention;
    a.hidden = (int64_t)mx.need("hidden_size"), a.num_heads = (int64_t)mx.need("num_heads");
    a.num_kv_heads = (int64_t)mx.need("num_kv_heads"), a.head_dim = (int64_t)mx.need("head_dim");
    a.window = (int64_t)mx.num("window", 0), a.pairing = (int64_t)pos.need("pairing_code");
    a.rotary_dim = (int64_t)pos.need("rotary_dim"), a.scale = mx.need("scale");
    a.qkv_weight = load.place(plan.param(l, "mixer", "qkv_weight"));
    a.qkv_bias = load.place(plan.param(l, "mixer", "qkv_bias"));
    a.out_weight = load.place(plan.param(l, "mixer", "out_weight"));
    a.out_bias = load.place(plan.param(l, "mixer", "out_bias"));
    auto table = plan.tables.find({l, "mixer"});
    if (table == plan.tables.end() || (int64_t)table->second.size() * 2 != a.rotary_dim) die("plan: layer without its table of angles");
    void* freq = nullptr;
    HIP_OK(hipMalloc(&freq, table->second.size() * 4 + 256));
    HIP_OK(hipMemcpy(freq, table->second.data(), table->second.size() * 4, hipMemcpyHostToDevice));
    a.inv_freq = (const float*)freq;
    if (ff.kind == "dense_swiglu") {
      d.ffn_kind = TQ_FFN_DENSE;
      d.dense.hidden = (int64_t)ff.need("hidden_size"), d.dense.inner = (int64_t)ff.need("inner_size");
      d.dense.gate = gate_code(ff.text("activation", "silu"));
      d.dense.gate_w = load.place(plan.param(l, "ffn", "gate"));
      d.dense.up_w = load.place(plan.param(l, "ffn", "up"));
      d.dense.down_w = load.place(plan.param(l, "ffn", "down"));
    } else if (ff.kind == "moe_swiglu") {
      d.ffn_kind = TQ_FFN_MOE;
      tq_moe_ffn_desc& m = d.moe;
      m.hidden = (int64_t)ff.need("hidden_size"), m.num_experts = (int64_t)ff.need("num_experts");
      m.top_k = (int64_t)ff.need("top_k"), m.inner = (int64_t)ff.need("expert_size");
      m.shared_inner = (int64_t)ff.num("shared_size", 0), m.renormalize = (int64_t)ff.num("renormalize", 0);
      m.gate = gate_code(ff.text("activation", "silu"));
      m.router = load.place(plan.param(l, "ffn", "router"));
      if (ff.num("shared_gated", 0) != 0) m.shared_scale = load.place(plan.param(l, "ffn", "shared_scale"));
      m.expert_gate = load.place(plan.param(l, "ffn", "expert_gate"));
      m.expert_up = load.place(plan.param(l, "ffn", "expert_up"));
      m.expert_down = load.place(plan.param(l, "ffn", "expert_down"));
      m.shared_gate = load.place(plan.param(l, "ffn", "shared_gate"));
      m.shared_up = load.place(plan.param(l, "ffn", "shared_up"));
      m.shared_down = load.place(plan.param(l, "ffn", "shared_down"));
    } else {
      die("layer " + std::to_string(l) + ": unknown feed-forward " + ff.kind);
    }
  }
  tq_model_desc model;
  memset(&model, 0, sizeof(model));
  model.vocab = V, model.hidden = H, model.n_layers = n_layers, model.n_entries = n_entries;
  model.embedding = load.place(plan.param(-1, "model", "embedding"));
  model.lm_head = plan.tied ? model.embedding : load.place(plan.param(-1, "model", "lm_head"));
  const PartLine& fin = plan.part(-1, "final_norm");
  model.final_norm = {load.place(plan.param(-1, "final_norm", "weight")), fin.need("eps")};
  model.embedding_scale = model_num("embedding_scale"), model.logit_softcap = model_num("logit_softcap");
  if (!load.missing.empty() || !load.wrong.empty()) {
    std::string msg = "checkpoint does not fit the model:";
    if (!load.missing.empty()) {
      msg += "\n  missing tensors (" + std::to_string(load.missing.size()) + "):";
      for (size_t i = 0; i < load.missing.size() && i < 20; ++i) msg += " " + load.missing[i];
    }
    if (!load.wrong.empty()) {
      msg += "\n  wrong shapes or types (" + std::to_string(load.wrong.size()) + "):";
      for (size_t i = 0; i < load.wrong.size() && i < 20; ++i) msg += " " + load.wrong[i];
    }
    die(msg);
  }
  fprintf(stderr, "tq_run: %s, %d layers, %.1f MB of parameters on the device (%s)\n", plan.architecture.c_str(), n_layers,
          load.placed / 1048576.0, plan.act.c_str());

  // the cache: a slot per prompt, pages of 64 positions, every entry's keys and values in pools of its own, the page
  // table the identity (slot s holds pages s * per_seq ..)
  const int B0 = (int)prompts.size(), page = 64;
  const int64_t max_positions = (int64_t)model_num("max_positions");
  size_t longest = 0;
  for (auto& p : prompts) longest = p.size() > longest ? p.size() : longest;
  int64_t reach = (int64_t)longest + max_new + 1;
  if (reach > max_positions) reach = max_positions;
  if ((int64_t)longest > max_positions) die("a prompt is longer than the model's " + std::to_string(max_positions) + " positions");
  const int per_seq = (int)((reach + page - 1) / page);
  std::vector<int> table_host((size_t)B0 * per_seq);
  for (int s = 0; s < B0; ++s)
    for (int p = 0; p < per_seq; ++p) table_host[(size_t)s * per_seq + p] = s * per_seq + p;
  int* table = nullptr;
  HIP_OK(hipMalloc((void**)&table, table_host.size() * 4 + 256));
  HIP_OK(hipMemcpy(table, table_host.data(), table_host.size() * 4, hipMemcpyHostToDevice));
  std::vector<tq_entry_desc> entries((size_t)n_entries);
  for (int e = 0; e < n_entries; ++e) {
    tq_entry_desc& d = entries[e];
    memset(&d, 0, sizeof(d));
    d.layer = plan.entries[e].first;
    const int of = plan.entries[e].second;
    const tq_attention_desc& a = layers[d.layer].attention;
    d.table = table, d.table_width = per_seq, d.layer_offset = 0, d.page_size = page;
    d.page_stride = a.num_kv_heads * page * a.head_dim;
    if (of >= 0) {
      if (of >= e) die("plan: an entry reads the cache of a later one");
      d.k_pages = entries[of].k_pages, d.v_pages = entries[of].v_pages, d.owns = 0;
      if (d.page_stride != entries[of].page_stride) die("plan: an entry reads a cache of other sizes");
    } else {
      const size_t bytes = (size_t)B0 * per_seq * d.page_stride * act_bytes;
      HIP_OK(hipMalloc(&d.k_pages, bytes + 256));
      HIP_OK(hipMalloc(&d.v_pages, bytes + 256));
      HIP_OK(hipMemset(d.k_pages, 0, bytes));      // rows behind a sequence's end are read (and masked): they hold numbers
      HIP_OK(hipMemset(d.v_pages, 0, bytes));
      d.owns = 1;
    }
  }
  model.layers = layers.data(), model.entries = entries.data();

  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  std::vector<int> length(B0, 0), live;
  std::vector<std::vector<int>> out(B0);
  std::vector<std::string> reason(B0);
  for (int s = 0; s < B0; ++s) live.push_back(s);
  std::vector<std::vector<int>> next = prompts;      // what each live sequence brings to the next step
  void* workspace = nullptr;
  size_t workspace_bytes = 0;
  int* ints = nullptr;
  size_t ints_cap = 0;
  float* logits = nullptr;
  int* chosen = nullptr;
  HIP_OK(hipMalloc((void**)&logits, (size_t)B0 * V * 4 + 256));
  HIP_OK(hipMalloc((void**)&chosen, (size_t)B0 * 4 + 256));
  while (!live.empty()) {
    const int B = (int)live.size();
    std::vector<int> tokens, positions, slot_of, cu(1, 0), slots, start, want;
    int max_new_here = 0, max_end = 0;
    for (int s : live) {
      const std::vector<int>& t = next[s];
      for (size_t j = 0; j < t.size(); ++j) {
        tokens.push_back(t[j]);
        positions.push_back(length[s] + (int)j);
        slot_of.push_back(s);
      }
      slots.push_back(s);
      start.push_back(length[s]);
      cu.push_back((int)tokens.size());
      want.push_back((int)tokens.size() - 1);
      max_new_here = (int)t.size() > max_new_here ? (int)t.size() : max_new_here;
      max_end = length[s] + (int)t.size() > max_end ? length[s] + (int)t.size() : max_end;
    }
    const int T = (int)tokens.size();
    std::vector<int> packed;
    for (const std::vector<int>* v : {&tokens, &positions, &slot_of, &cu, &slots, &start, &want}) packed.insert(packed.end(), v->begin(), v->end());
    if (packed.size() > ints_cap) {
      if (ints) HIP_OK(hipFree(ints));
      ints_cap = packed.size() * 2;
      HIP_OK(hipMalloc((void**)&ints, ints_cap * 4 + 256));
    }
    HIP_OK(hipMemcpyAsync(ints, packed.data(), packed.size() * 4, hipMemcpyHostToDevice, stream));
    tq_step_desc step;
    memset(&step, 0, sizeof(step));
    step.T = T, step.B = B, step.n_want = B, step.max_new = max_new_here, step.max_end = max_end, step.decode = max_new_here == 1;
    step.expert_128_from = step.expert_256_from = 1 << 30, step.expert_pairs_from = 48, step.side_from = 1 << 30;      // own kernels for every product, one stream
    step.tokens = ints, step.positions = ints + T, step.slot_of_token = ints + 2 * T, step.cu_seqlens = ints + 3 * T;
    step.slots = ints + 3 * T + B + 1, step.start = ints + 3 * T + 2 * B + 1, step.want_rows = ints + 3 * T + 3 * B + 1;
    step.logits = logits, step.stream = stream;
    const int64_t need = step_workspace(&model, &step);
    if (need < 0) die(std::string("step executor: ") + last_error());
    if ((size_t)need > workspace_bytes) {
      if (workspace) HIP_OK(hipFree(workspace));
      workspace_bytes = (size_t)need;
      HIP_OK(hipMalloc(&workspace, workspace_bytes + 256));
    }
    step.workspace = workspace, step.workspace_bytes = (int64_t)workspace_bytes;
    if (step_forward(&model, &step) != 0) die(std::string("step executor: ") + last_error());
    if (argmax(logits, B, (int)V, chosen, stream) != 0) die("tq_argmax failed");
    std::vector<int> picked((size_t)B);
    HIP_OK(hipMemcpyAsync(picked.data(), chosen, (size_t)B * 4, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<int> going;
    for (int i = 0; i < B; ++i) {
      const int s = live[i], tok = picked[i];
      length[s] += (int)next[s].size();
      bool stop = false;
      for (int t : plan.stop) stop = stop || t == tok;
      if (stop) {
        reason[s] = "stop";         // the end token is not emitted
        continue;
      }
      out[s].push_back(tok);
      if ((int)out[s].size() >= max_new) {
        reason[s] = "length";
      } else if ((int64_t)prompts[s].size() + (int64_t)out[s].size() >= max_positions) {
        reason[s] = "context";
      } else {
        next[s] = {tok};
        going.push_back(s);
      }
    }
    live = going;
  }
  for (int s = 0; s < B0; ++s) {
    printf("[%d]", s);
    for (int t : out[s]) printf(" %d", t);
    printf("  (%s)\n", reason[s].c_str());
  }
  return 0;
}
