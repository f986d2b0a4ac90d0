#include "proto.hpp"

#include <cctype>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>

namespace caffe {

// ---------------------------------------------------------------------------
// Message
// ---------------------------------------------------------------------------

int Message::count(const std::string& name) const {
  int n = 0;
  for (const auto& f : fields_) n += f.name == name;
  return n;
}

const Message::Field* Message::find(const std::string& name, int idx) const {
  for (const auto& f : fields_) {
    if (f.name == name && idx-- == 0) return &f;
  }
  return nullptr;
}

const Message& Message::sub(const std::string& name, int idx) const {
  static const Message kEmpty;
  const Field* f = find(name, idx);
  return (f && f->msg) ? *f->msg : kEmpty;
}

Message* Message::add_sub(const std::string& name) {
  Field f;
  f.name = name;
  f.msg = std::make_shared<Message>();
  fields_.push_back(f);
  return fields_.back().msg.get();
}

long Message::get_int(const std::string& name, long def, int idx) const {
  const Field* f = find(name, idx);
  if (!f) return def;
  char* end = nullptr;
  const long v = std::strtol(f->text.c_str(), &end, 0);
  if (end == f->text.c_str() || (*end != '\0' && *end != '.')) {
    // allow "3.0" style and reject identifiers
    const double d = std::strtod(f->text.c_str(), &end);
    CHECK(end != f->text.c_str() && *end == '\0')
        << "field '" << name << "': expected an integer, got '" << f->text << "'";
    return static_cast<long>(d);
  }
  return v;
}

double Message::get_float(const std::string& name, double def, int idx) const {
  const Field* f = find(name, idx);
  if (!f) return def;
  std::string t = f->text;
  if (!t.empty() && (t.back() == 'f' || t.back() == 'F') && t != "inf" && t != "-inf") t.pop_back();
  char* end = nullptr;
  const double d = std::strtod(t.c_str(), &end);
  CHECK(end != t.c_str() && *end == '\0')
      << "field '" << name << "': expected a number, got '" << f->text << "'";
  return d;
}

bool Message::get_bool(const std::string& name, bool def, int idx) const {
  const Field* f = find(name, idx);
  if (!f) return def;
  const std::string& t = f->text;
  if (t == "true" || t == "True" || t == "t" || t == "1") return true;
  if (t == "false" || t == "False" || t == "f" || t == "0") return false;
  LOG(FATAL) << "field '" << name << "': expected a bool, got '" << t << "'";
  return def;
}

std::string Message::get_string(const std::string& name, const std::string& def, int idx) const {
  const Field* f = find(name, idx);
  return f ? f->text : def;
}

void Message::add(const std::string& name, const std::string& text, bool quoted) {
  Field f;
  f.name = name;
  f.text = text;
  f.quoted = quoted;
  fields_.push_back(f);
}

void Message::add_int(const std::string& name, long v) { add(name, std::to_string(v)); }

void Message::add_float(const std::string& name, double v) {
  char buf[64];
  snprintf(buf, sizeof(buf), "%.9g", v);
  add(name, buf);
}

void Message::remove(const std::string& name) {
  std::vector<Field> kept;
  for (auto& f : fields_)
    if (f.name != name) kept.push_back(std::move(f));
  fields_.swap(kept);
}

void Message::set(const std::string& name, const std::string& text, bool quoted) {
  remove(name);
  add(name, text, quoted);
}

std::string Message::DebugString(int indent) const {
  std::ostringstream os;
  const std::string pad(indent, ' ');
  for (const auto& f : fields_) {
    if (f.msg) {
      os << pad << f.name << " {\n" << f.msg->DebugString(indent + 2) << pad << "}\n";
    } else if (f.floats) {
      for (float v : *f.floats) {
        char buf[64];
        snprintf(buf, sizeof(buf), "%.9g", v);
        os << pad << f.name << ": " << buf << "\n";
      }
    } else if (f.quoted) {
      os << pad << f.name << ": \"";
      for (char c : f.text) {
        if (c == '"' || c == '\\') os << '\\';
        if (c == '\n') os << "\\n";
        else os << c;
      }
      os << "\"\n";
    } else {
      os << pad << f.name << ": " << f.text << "\n";
    }
  }
  return os.str();
}

// ---------------------------------------------------------------------------
// Text format
// ---------------------------------------------------------------------------

namespace {

class TextParser {
 public:
  TextParser(const char* data, size_t len) : p_(data), end_(data + len), line_(1), bol_(data) {}

  void ParseMessage(Message* out, char closer) {
    for (;;) {
      SkipSpace();
      if (p_ >= end_) {
        if (closer != 0) Fail("unexpected end of input, missing closing brace");
        return;
      }
      if (*p_ == closer && closer != 0) {
        ++p_;
        return;
      }
      if (*p_ == '}' || *p_ == '>') Fail("unbalanced closing brace");
      const std::string name = ReadIdentifier();
      SkipSpace();
      bool colon = false;
      if (p_ < end_ && *p_ == ':') {
        colon = true;
        ++p_;
        SkipSpace();
      }
      if (p_ < end_ && (*p_ == '{' || *p_ == '<')) {
        const char close = *p_ == '{' ? '}' : '>';
        ++p_;
        ParseMessage(out->add_sub(name), close);
      } else {
        if (!colon) Fail("expected ':' or '{' after field name '" + name + "'");
        if (p_ < end_ && *p_ == '[') {
          ++p_;
          for (;;) {
            SkipSpace();
            if (p_ < end_ && *p_ == ']') {
              ++p_;
              break;
            }
            ReadScalar(name, out);
            SkipSpace();
            if (p_ < end_ && *p_ == ',') ++p_;
          }
        } else {
          ReadScalar(name, out);
        }
      }
      SkipSpace();
      if (p_ < end_ && (*p_ == ',' || *p_ == ';')) ++p_;
    }
  }

 private:
  void Fail(const std::string& what) {
    LOG(FATAL) << "prototxt parse error at " << line_ << ":" << (p_ - bol_ + 1) << ": " << what;
  }

  void SkipSpace() {
    while (p_ < end_) {
      if (*p_ == '\n') {
        ++line_;
        bol_ = p_ + 1;
        ++p_;
      } else if (isspace(static_cast<unsigned char>(*p_))) {
        ++p_;
      } else if (*p_ == '#') {
        while (p_ < end_ && *p_ != '\n') ++p_;
      } else {
        break;
      }
    }
  }

  std::string ReadIdentifier() {
    const char* s = p_;
    if (p_ < end_ && *p_ == '[') {  // extension syntax [a.b.c]
      while (p_ < end_ && *p_ != ']') ++p_;
      if (p_ < end_) ++p_;
      return std::string(s, p_);
    }
    while (p_ < end_ && (isalnum(static_cast<unsigned char>(*p_)) || *p_ == '_' || *p_ == '.')) ++p_;
    if (p_ == s) Fail(std::string("expected a field name, got '") + *p_ + "'");
    return std::string(s, p_);
  }

  void ReadScalar(const std::string& name, Message* out) {
    if (p_ >= end_) Fail("missing value for '" + name + "'");
    if (*p_ == '"' || *p_ == '\'') {
      std::string v;
      // adjacent string literals concatenate
      while (p_ < end_ && (*p_ == '"' || *p_ == '\'')) {
        const char q = *p_++;
        while (p_ < end_ && *p_ != q) {
          if (*p_ == '\n') Fail("newline inside string");
          if (*p_ == '\\' && p_ + 1 < end_) {
            ++p_;
            switch (*p_) {
              case 'n': v += '\n'; break;
              case 't': v += '\t'; break;
              case 'r': v += '\r'; break;
              case '0': v += '\0'; break;
              default: v += *p_; break;
            }
            ++p_;
          } else {
            v += *p_++;
          }
        }
        if (p_ >= end_) Fail("unterminated string");
        ++p_;
        SkipSpace();
      }
      out->add(name, v, true);
      return;
    }
    const char* s = p_;
    while (p_ < end_ && !isspace(static_cast<unsigned char>(*p_)) && *p_ != ',' && *p_ != ';' &&
           *p_ != '}' && *p_ != '>' && *p_ != ']' && *p_ != '#' && *p_ != '{')
      ++p_;
    if (p_ == s) Fail("missing value for '" + name + "'");
    out->add(name, std::string(s, p_));
  }

  const char* p_;
  const char* end_;
  int line_;
  const char* bol_;
};

}  // namespace

void ParseText(const char* data, size_t len, Message* out) {
  TextParser parser(data, len);
  parser.ParseMessage(out, 0);
}

// ---------------------------------------------------------------------------
// Wire format
// ---------------------------------------------------------------------------

namespace {

enum WireKind { W_INT, W_FLOAT, W_DOUBLE, W_STRING, W_MESSAGE, W_FLOATS, W_DOUBLES };

struct WireField {
  int number;
  const char* name;
  WireKind kind;
  const struct WireSchema* sub;
};

struct WireSchema {
  const WireField* fields;
  int n;
};

// caffe.proto:6-8
const WireField kBlobShapeFields[] = {{1, "dim", W_INT, nullptr}};
const WireSchema kBlobShape = {kBlobShapeFields, 1};
// caffe.proto:10-22
const WireField kBlobProtoFields[] = {
    {1, "num", W_INT, nullptr},      {2, "channels", W_INT, nullptr},
    {3, "height", W_INT, nullptr},   {4, "width", W_INT, nullptr},
    {5, "data", W_FLOATS, nullptr},  {7, "shape", W_MESSAGE, &kBlobShape},
    {8, "double_data", W_DOUBLES, nullptr}};
const WireSchema kBlobProto = {kBlobProtoFields, 7};
// caffe.proto:143-233 (identity, wiring and weights; *_param messages of a
// trained model are not needed to copy its weights and are skipped)
const WireField kLayerFields[] = {{1, "name", W_STRING, nullptr},
                                  {2, "type", W_STRING, nullptr},
                                  {3, "bottom", W_STRING, nullptr},
                                  {4, "top", W_STRING, nullptr},
                                  {7, "blobs", W_MESSAGE, &kBlobProto}};
const WireSchema kLayer = {kLayerFields, 5};
// V1LayerParameter (caffe.proto V1LayerParameter: name = 4, blobs = 6)
const WireField kV1LayerFields[] = {{4, "name", W_STRING, nullptr},
                                    {6, "blobs", W_MESSAGE, &kBlobProto}};
const WireSchema kV1Layer = {kV1LayerFields, 2};
// caffe.proto:51-83
const WireField kNetFields[] = {{1, "name", W_STRING, nullptr},
                                {2, "layers", W_MESSAGE, &kV1Layer},
                                {100, "layer", W_MESSAGE, &kLayer}};
const WireSchema kNet = {kNetFields, 3};

class WireReader {
 public:
  WireReader(const uint8_t* p, const uint8_t* end) : p_(p), end_(end) {}

  void Parse(const WireSchema& schema, Message* out) {
    while (p_ < end_) {
      const uint64_t key = Varint();
      const int number = static_cast<int>(key >> 3);
      const int wt = static_cast<int>(key & 7);
      const WireField* wf = nullptr;
      for (int i = 0; i < schema.n; ++i)
        if (schema.fields[i].number == number) wf = &schema.fields[i];
      if (!wf) {
        Skip(wt);
        continue;
      }
      switch (wf->kind) {
        case W_INT:
          if (wt == 2) {  // packed
            const uint8_t* stop = Sub();
            while (p_ < stop) out->add_int(wf->name, static_cast<long>(Varint()));
          } else {
            Expect(wt, 0);
            out->add_int(wf->name, static_cast<long>(Varint()));
          }
          break;
        case W_FLOAT:
          Expect(wt, 5);
          out->add_float(wf->name, Fixed32());
          break;
        case W_DOUBLE:
          Expect(wt, 1);
          out->add_float(wf->name, Fixed64());
          break;
        case W_STRING: {
          Expect(wt, 2);
          const uint8_t* stop = Sub();
          out->add(wf->name, std::string(reinterpret_cast<const char*>(p_), stop - p_), true);
          p_ = stop;
          break;
        }
        case W_MESSAGE: {
          Expect(wt, 2);
          const uint8_t* stop = Sub();
          WireReader inner(p_, stop);
          inner.Parse(*wf->sub, out->add_sub(wf->name));
          p_ = stop;
          break;
        }
        case W_FLOATS:
        case W_DOUBLES: {
          // One bulk payload per blob; repeated chunks append.
          Message::Field* dst = nullptr;
          for (auto& f : out->fields())
            if (f.name == "data" && f.floats) dst = &f;
          if (!dst) {
            Message::Field f;
            f.name = "data";
            f.floats = std::make_shared<std::vector<float> >();
            out->fields().push_back(f);
            dst = &out->fields().back();
          }
          const bool is_double = wf->kind == W_DOUBLES;
          if (wt == 2) {
            const uint8_t* stop = Sub();
            const size_t width = is_double ? 8 : 4;
            const size_t n = (stop - p_) / width;
            CHECK_EQ((stop - p_) % width, 0u) << "truncated packed array in caffemodel";
            const size_t old = dst->floats->size();
            dst->floats->resize(old + n);
            if (!is_double) {
              memcpy(dst->floats->data() + old, p_, n * 4);
            } else {
              for (size_t i = 0; i < n; ++i) {
                double d;
                memcpy(&d, p_ + 8 * i, 8);
                (*dst->floats)[old + i] = static_cast<float>(d);
              }
            }
            p_ = stop;
          } else if (is_double) {
            Expect(wt, 1);
            dst->floats->push_back(static_cast<float>(Fixed64()));
          } else {
            Expect(wt, 5);
            dst->floats->push_back(Fixed32());
          }
          break;
        }
      }
    }
  }

 private:
  void Expect(int got, int want) {
    CHECK_EQ(got, want) << "caffemodel: unexpected wire type";
  }
  uint64_t Varint() {
    uint64_t v = 0;
    for (int shift = 0; shift < 64; shift += 7) {
      CHECK(p_ < end_) << "caffemodel: truncated varint";
      const uint8_t b = *p_++;
      v |= static_cast<uint64_t>(b & 0x7f) << shift;
      if (!(b & 0x80)) return v;
    }
    LOG(FATAL) << "caffemodel: malformed varint";
    return 0;
  }
  float Fixed32() {
    CHECK(end_ - p_ >= 4) << "caffemodel: truncated fixed32";
    float f;
    memcpy(&f, p_, 4);
    p_ += 4;
    return f;
  }
  double Fixed64() {
    CHECK(end_ - p_ >= 8) << "caffemodel: truncated fixed64";
    double d;
    memcpy(&d, p_, 8);
    p_ += 8;
    return d;
  }
  // Reads a length prefix and returns the end of that sub-range.
  const uint8_t* Sub() {
    const uint64_t n = Varint();
    CHECK(static_cast<uint64_t>(end_ - p_) >= n) << "caffemodel: truncated length-delimited field";
    return p_ + n;
  }
  void Skip(int wt) {
    switch (wt) {
      case 0: Varint(); break;
      case 1: CHECK(end_ - p_ >= 8) << "caffemodel: truncated"; p_ += 8; break;
      case 2: p_ = Sub(); break;
      case 5: CHECK(end_ - p_ >= 4) << "caffemodel: truncated"; p_ += 4; break;
      default: LOG(FATAL) << "caffemodel: unsupported wire type " << wt;
    }
  }

  const uint8_t* p_;
  const uint8_t* end_;
};

std::string ReadFile(const std::string& file, const char* what) {
  std::ifstream in(file, std::ios::binary);
  CHECK(in.good()) << "File not found: " << file << " (" << what << ")";
  std::ostringstream ss;
  ss << in.rdbuf();
  return ss.str();
}

void PutVarint(std::string* s, uint64_t v) {
  while (v >= 0x80) {
    s->push_back(static_cast<char>((v & 0x7f) | 0x80));
    v >>= 7;
  }
  s->push_back(static_cast<char>(v));
}
void PutKey(std::string* s, int number, int wt) { PutVarint(s, (uint64_t)number << 3 | wt); }
void PutBytes(std::string* s, int number, const std::string& bytes) {
  PutKey(s, number, 2);
  PutVarint(s, bytes.size());
  s->append(bytes);
}

}  // namespace

void ParseBinaryNet(const uint8_t* data, size_t len, Message* out) {
  WireReader reader(data, data + len);
  reader.Parse(kNet, out);
}

std::string SerializeBinaryNet(const Message& net) {
  std::string out;
  if (net.has("name")) PutBytes(&out, 1, net.get_string("name"));
  for (const auto& lf : net.fields()) {
    if (lf.name != "layer" || !lf.msg) continue;
    std::string layer;
    PutBytes(&layer, 1, lf.msg->get_string("name"));
    PutBytes(&layer, 2, lf.msg->get_string("type"));
    for (const auto& bf : lf.msg->fields()) {
      if (bf.name != "blobs" || !bf.msg) continue;
      std::string blob, shape, dims;
      const Message& sh = bf.msg->sub("shape");
      for (int i = 0; i < sh.count("dim"); ++i) PutVarint(&dims, sh.get_int("dim", 0, i));
      PutBytes(&shape, 1, dims);
      const Message::Field* data = nullptr;
      for (const auto& f : bf.msg->fields())
        if (f.name == "data" && f.floats) data = &f;
      if (data) {
        std::string raw(reinterpret_cast<const char*>(data->floats->data()),
                        data->floats->size() * 4);
        PutBytes(&blob, 5, raw);
      }
      PutBytes(&blob, 7, shape);
      PutBytes(&layer, 7, blob);
    }
    PutBytes(&out, 100, layer);
  }
  return out;
}

void ReadNetParamsFromTextFileOrDie(const std::string& file, NetParameter* param) {
  const std::string text = ReadFile(file, "network prototxt");
  ParseText(text.data(), text.size(), param);
  UpgradeNetAsNeeded(file, param);
}

void ReadNetParamsFromBinaryFileOrDie(const std::string& file, NetParameter* param) {
  const std::string bytes = ReadFile(file, "caffemodel");
  ParseBinaryNet(reinterpret_cast<const uint8_t*>(bytes.data()), bytes.size(), param);
}

namespace {

// V1LayerParameter.LayerType -> type string (reference src/util/upgrade_proto.cpp:215-265;
// enum values from caffe.proto's V1LayerParameter).  A text file names the enum
// by identifier; the number is accepted as well.
struct V1Type {
  const char* ident;
  int number;
  const char* type;
};
const V1Type kV1Types[] = {
    {"NONE", 0, ""},
    {"ABSVAL", 35, "AbsVal"},
    {"BNLL", 2, "BNLL"},
    {"CONCAT", 3, "Concat"},
    {"CONVOLUTION", 4, "Convolution"},
    {"DECONVOLUTION", 39, "Deconvolution"},
    {"DROPOUT", 6, "Dropout"},
    {"ELTWISE", 25, "Eltwise"},
    {"EXP", 38, "Exp"},
    {"FLATTEN", 8, "Flatten"},
    {"INNER_PRODUCT", 14, "InnerProduct"},
    {"LRN", 15, "LRN"},
    {"MVN", 34, "MVN"},
    {"POOLING", 17, "Pooling"},
    {"POWER", 26, "Power"},
    {"RELU", 18, "ReLU"},
    {"SIGMOID", 19, "Sigmoid"},
    {"SOFTMAX", 20, "Softmax"},
    {"SPLIT", 22, "Split"},
    {"SLICE", 33, "Slice"},
    {"TANH", 23, "TanH"},
    {"THRESHOLD", 31, "Threshold"},
};

// The fields of a V1 layer that UpgradeV1LayerParameter carries over and that
// matter to a forward pass (reference src/util/upgrade_proto.cpp:86-213); the
// learning-rate, weight-decay, loss-weight and parameter-sharing fields have no
// reader in this library and are dropped.
const char* const kV1Carried[] = {
    "bottom", "top", "name", "include", "exclude", "blobs", "concat_param", "convolution_param",
    "dropout_param", "eltwise_param", "exp_param", "inner_product_param", "lrn_param", "mvn_param",
    "pooling_param", "power_param", "relu_param", "sigmoid_param", "softmax_param", "slice_param",
    "tanh_param", "threshold_param"};

void UpgradeV1Net(const std::string& source, NetParameter* param) {
  CHECK(!param->has("layer"))
      << source << ": Refusing to upgrade inconsistent NetParameter input; the definition "
      << "includes both 'layer' and 'layers' fields. The current format defines 'layer' fields "
      << "with string type like layer { type: 'Layer' ... } and not layers { type: LAYER ... }. "
      << "Manually switch the definition to 'layer' format to continue.";
  for (auto& f : param->fields()) {
    if (f.name != "layers" || !f.msg) continue;
    const Message& v1 = *f.msg;
    auto layer = std::make_shared<Message>();
    for (const auto& g : v1.fields()) {
      bool carried = false;
      for (const char* k : kV1Carried) carried = carried || g.name == k;
      if (carried) layer->fields().push_back(g);
    }
    if (v1.has("type")) {
      const Message::Field* t = v1.find("type");
      const char* mapped = nullptr;
      for (const V1Type& e : kV1Types)
        if (t->text == e.ident || t->text == std::to_string(e.number)) mapped = e.type;
      CHECK(mapped && !t->quoted)
          << source << ": Unknown V1LayerParameter layer type: " << t->text;
      layer->add("type", mapped, true);
    }
    f.name = "layer";
    f.msg = layer;
  }
}

}  // namespace

void UpgradeNetAsNeeded(const std::string& source, NetParameter* param) {
  if (param->has("layers")) UpgradeV1Net(source, param);
  if (!param->has("input")) return;
  // `input: "data"` + (`input_shape {dim..}` | 4 x `input_dim`) -> Input layer.
  const int n_in = param->count("input");
  const bool has_shape = param->has("input_shape");
  const bool has_dim = param->has("input_dim");
  CHECK(has_shape || has_dim) << source << ": net declares inputs without shapes";
  auto layer = std::make_shared<Message>();
  layer->add("name", "input", true);
  layer->add("type", "Input", true);
  Message* ip = nullptr;
  for (int i = 0; i < n_in; ++i) layer->add("top", param->get_string("input", "", i), true);
  ip = layer->add_sub("input_param");
  if (has_shape) {
    CHECK(param->count("input_shape") == n_in || param->count("input_shape") == 1)
        << source << ": need one input_shape per input";
    for (int i = 0; i < param->count("input_shape"); ++i) {
      Message* shape = ip->add_sub("shape");
      const Message& src = param->sub("input_shape", i);
      for (int d = 0; d < src.count("dim"); ++d) shape->add_int("dim", src.get_int("dim", 0, d));
    }
  } else {
    CHECK_EQ(param->count("input_dim"), 4 * n_in) << source << ": need 4 input_dim per input";
    for (int i = 0; i < n_in; ++i) {
      Message* shape = ip->add_sub("shape");
      for (int d = 0; d < 4; ++d) shape->add_int("dim", param->get_int("input_dim", 0, 4 * i + d));
    }
  }
  param->remove("input");
  param->remove("input_shape");
  param->remove("input_dim");
  Message::Field f;
  f.name = "layer";
  f.msg = layer;
  // the Input layer must come first
  auto& fields = param->fields();
  auto it = fields.begin();
  while (it != fields.end() && it->name != "layer") ++it;
  fields.insert(it, f);
}

}  // namespace caffe
