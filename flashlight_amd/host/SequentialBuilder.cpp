#include "SequentialBuilder.h"

#include <fstream>
#include <sstream>
#include <stdexcept>

namespace fl {
namespace pkg {
namespace runtime {
namespace {

std::string trim(const std::string& s) {
  const char* ws = " \t\r\n";
  const size_t a = s.find_first_not_of(ws);
  if (a == std::string::npos) return "";
  return s.substr(a, s.find_last_not_of(ws) - a + 1);
}

void replaceAll(std::string& s, const std::string& from, const std::string& to) {
  for (size_t pos = 0; (pos = s.find(from, pos)) != std::string::npos; pos += to.size()) s.replace(pos, from.size(), to);
}

std::vector<std::string> splitOnWhitespace(const std::string& s) {
  std::istringstream in(s);
  std::vector<std::string> out;
  for (std::string tok; in >> tok;) out.push_back(tok);
  return out;
}

[[noreturn]] void failParse(const std::string& line) { throw std::invalid_argument("Failed parsing - " + line); }

int toInt(const std::string& s, const std::string& line) {
  try {
    size_t used = 0;
    const int v = std::stoi(s, &used);
    if (used != s.size()) failParse(line);
    return v;
  } catch (const std::invalid_argument&) {
    failParse(line);
  } catch (const std::out_of_range&) {
    failParse(line);
  }
}

// one module from one line (SequentialBuilder.cpp:98-640)
ModulePtr parseLine(const std::string& line) {
  const std::vector<std::string> p = splitOnWhitespace(line);
  if (p.empty()) failParse(line);
  const size_t n = p.size();
  auto inRange = [&](size_t a, size_t c) { return a <= n && n <= c; };
  auto I = [&](size_t i) { return toInt(p[i], line); };
  const std::string& op = p[0];
  auto F = [&](size_t i) {
    try {
      return std::stod(p[i]);
    } catch (const std::exception&) {
      failParse(line);
    }
    return 0.0;
  };

  if (op == "V" || op == "RO") {                 // SequentialBuilder.cpp:116-129
    if (n < 2) failParse(line);
    std::vector<Dim> dims;
    for (size_t i = 1; i < n; ++i) dims.push_back(I(i));
    if (op == "RO") return std::make_shared<Reorder>(Shape(dims));
    return std::make_shared<View>(Shape(dims));
  }
  if (op == "C" || op == "C1") {
    if (!inRange(5, 7)) failParse(line);
    const int px = n >= 6 ? I(5) : 0, dx = n >= 7 ? I(6) : 1;
    return std::make_shared<Conv2D>(I(1), I(2), I(3), 1, I(4), 1, px, 0, dx, 1);
  }
  if (op == "TDS") {                              // SequentialBuilder.cpp:228-243
    if (!inRange(4, 8)) failParse(line);
    const double dropprob = n >= 5 ? F(4) : 0.0;
    const int l2 = n >= 6 ? I(5) : 0, rPad = n >= 7 ? I(6) : -1;
    const bool lNormIncludeTime = !(n >= 8 && I(7) == 0);
    return std::make_shared<TDSBlock>(I(1), I(2), I(3), dropprob, l2, rPad, lNormIncludeTime);
  }
  if (op == "AC") {                               // :245-258
    if (!inRange(5, 8)) failParse(line);
    const int px = n >= 6 ? I(5) : 0, dx = n >= 8 ? I(7) : 1;
    const float future = n >= 7 ? (float)F(6) : 1.0f;
    return std::make_shared<AsymmetricConv1D>(I(1), I(2), I(3), I(4), px, future, dx);
  }
  if (op == "C2") {
    if (!inRange(7, 11)) failParse(line);
    const int px = n >= 8 ? I(7) : 0, py = n >= 9 ? I(8) : 0, dx = n >= 10 ? I(9) : 1, dy = n >= 11 ? I(10) : 1;
    return std::make_shared<Conv2D>(I(1), I(2), I(3), I(4), I(5), I(6), px, py, dx, dy);
  }
  if (op == "L") {
    if (!inRange(3, 4)) failParse(line);
    const bool bias = !(n == 4 && p[3] == "0");
    return std::make_shared<Linear>(I(1), I(2), bias);
  }
  if (op == "BN") {
    if (!inRange(3, 5)) failParse(line);
    std::vector<int> axes;
    for (size_t i = 2; i < n; ++i) axes.push_back(I(i));
    return std::make_shared<BatchNorm>(axes, I(1));
  }
  if (op == "LN") {
    if (!inRange(2, 4)) failParse(line);
    std::vector<int> axes;
    for (size_t i = 1; i < n; ++i) axes.push_back(I(i));
    // the reference rejects the pre-2020 spelling "LN 3" (SequentialBuilder.cpp:340-349)
    if (axes == std::vector<int>{3}) failParse(line);
    return std::make_shared<LayerNorm>(axes);
  }
  if (op == "M" || op == "A") {
    if (n < 5) failParse(line);
    const int px = n > 5 ? I(5) : 0, py = n > 6 ? I(6) : 0;
    return std::make_shared<Pool2D>(I(1), I(2), I(3), I(4), px, py,
                                    op == "A" ? PoolingMode::AVG_INCLUDE_PADDING : PoolingMode::MAX);
  }
  if (op == "R") {
    if (n != 1) failParse(line);
    return std::make_shared<ReLU>();
  }
  if (op == "LSM") {
    if (n != 2) failParse(line);
    return std::make_shared<LogSoftmax>(I(1));
  }
  // the other activations (SequentialBuilder.cpp:390-466) and dropout (:360-366)
  if (op == "ELU" || op == "R6" || op == "LG" || op == "HT" || op == "T") {
    if (n != 1) failParse(line);
    if (op == "ELU") return std::make_shared<ELU>();
    if (op == "R6") return std::make_shared<ReLU6>();
    if (op == "LG") return std::make_shared<Log>();
    if (op == "HT") return std::make_shared<HardTanh>();
    return std::make_shared<Tanh>();
  }
  if (op == "E") {                                   // :291-298
    if (n != 3) failParse(line);
    return std::make_shared<Embedding>(I(1), I(2));
  }
  if (op == "PR") {                                  // :411-418
    if (n < 1 || n > 3) failParse(line);
    return std::make_shared<PReLU>(n > 1 ? I(1) : 1, n > 2 ? F(2) : 0.25);
  }
  if (op == "GLU") {
    if (n != 2) failParse(line);
    return std::make_shared<GatedLinearUnit>(I(1));
  }
  if (op == "SH") {
    if (!inRange(1, 2)) failParse(line);
    return std::make_shared<Swish>(n > 1 ? (double)(float)F(1) : 1.0);      // std::stof there
  }
  if (op == "DO") {
    if (n != 2) failParse(line);
    return std::make_shared<Dropout>(F(1));
  }
  if (op == "PC") {                               // SequentialBuilder.cpp:583-589; the names of fl::stringToDtype that
    if (n != 2) failParse(line);                  // this backend converts among, and bf16
    if (p[1] == "f32") return std::make_shared<PrecisionCast>(dtype::f32);
    if (p[1] == "f16") return std::make_shared<PrecisionCast>(dtype::f16);
    if (p[1] == "bf16") return std::make_shared<PrecisionCast>(dtype::bf16);
    throw std::invalid_argument("stringToDtype: Invalid input type: " + p[1]);
  }
  if (op == "PD") {                               // SequentialBuilder.cpp:131-144: a value, then (before, after) pairs
    if (!inRange(4, 10) || (n & 1)) failParse(line);
    const double val = F(1);
    std::vector<std::pair<int, int>> pads(4, {0, 0});
    for (size_t i = 2; i + 1 < n; i += 2) pads[(i - 2) / 2] = {I(i), I(i + 1)};
    return std::make_shared<Padding>(pads, val);
  }
  if (op == "WN") {                               // :352-359: a dimension, then the line of the wrapped module
    if (n < 3) failParse(line);
    std::string child;
    for (size_t i = 2; i < n; ++i) child += (i > 2 ? " " : "") + p[i];
    return std::make_shared<WeightNorm>(parseLine(child), I(1));
  }
  if (op == "RNN" || op == "GRU" || op == "LSTM") {
    if (n < 3) failParse(line);
    const RnnMode mode = op == "RNN" ? RnnMode::RELU : op == "GRU" ? RnnMode::GRU : RnnMode::LSTM;
    const int layers = n > 3 ? I(3) : 1;
    const bool bidirectional = n > 4 ? I(4) > 0 : false;
    const float dropout = n > 5 ? std::stof(p[5]) : 0.0f;
    return std::make_shared<RNN>(I(1), I(2), layers, mode, bidirectional, dropout);
  }
  static const char* const absent[] = {"TR", "CFR", "POSEMB", "SINPOSEMB", "ADAPTIVEE", "SAUG"};
  for (const char* a : absent)
    if (op == a)
      throw std::invalid_argument("buildSequentialModule: module '" + op +
                                  "' is not provided by this backend - " + line);
  failParse(line);
}

// The module that starts at lines[idx]; *parsed = the lines it took beyond its first (SequentialBuilder.cpp:98-104,
// 498-566): a residual block "RES layers skips [repeats]" is followed by its layer lines and its "SKIP from to [scale]" /
// "SKIPL from to projectionLayers [scale]" lines (the latter followed by the lines of the projection).
ModulePtr parseLines(const std::vector<std::string>& lines, size_t idx, size_t* parsed) {
  const std::string& line = lines[idx];
  *parsed = 0;
  const std::vector<std::string> p = splitOnWhitespace(line);
  if (p.empty()) failParse(line);
  if (p[0] == "SKIP" || p[0] == "SKIPL") failParse(line);      // only inside a residual block
  if (p[0] != "RES") return parseLine(line);
  if (p.size() <= 3) failParse(line);                          // :500-502: the number of repeats is not optional
  const int numResLayers = toInt(p[1], line), numSkip = toInt(p[2], line);
  const int numBlocks = p.size() == 4 ? toInt(p[3], line) : 1;
  if (numBlocks <= 0) throw std::invalid_argument("Invalid number of residual blocks: " + std::to_string(numBlocks));
  size_t taken = 0;
  auto block = [&]() {
    auto res = std::make_shared<Residual>();
    size_t projections = 0;
    for (int i = 1; i <= numResLayers + numSkip; ++i) {
      const size_t at = idx + (size_t)i + projections;
      if (at >= lines.size()) throw std::invalid_argument("Failed parsing Residual block");
      const std::string& rl = lines[at];
      const std::vector<std::string> q = splitOnWhitespace(rl);
      if (q.empty()) failParse(rl);
      if (q[0] == "SKIP") {
        if (q.size() < 3 || q.size() > 4) failParse(rl);
        res->addShortcut(toInt(q[1], rl), toInt(q[2], rl));
        if (q.size() == 4) res->addScale(toInt(q[2], rl), std::stof(q[3]));
      } else if (q[0] == "SKIPL") {
        if (q.size() < 4 || q.size() > 5) failParse(rl);
        const int nproj = toInt(q[3], rl);
        auto projection = std::make_shared<Sequential>();
        for (int j = 1; j <= nproj; ++j) {
          if (at + (size_t)j >= lines.size()) throw std::invalid_argument("Failed parsing Residual block");
          projection->add(parseLine(lines[at + (size_t)j]));
        }
        res->addShortcut(toInt(q[1], rl), toInt(q[2], rl), ModulePtr(projection));
        if (q.size() == 5) res->addScale(toInt(q[2], rl), std::stof(q[4]));
        projections += (size_t)nproj;
      } else {
        res->add(parseLine(rl));
      }
    }
    taken = (size_t)(numResLayers + numSkip) + projections;
    return res;
  };
  ModulePtr out;
  if (numBlocks > 1) {
    auto seq = std::make_shared<Sequential>();
    for (int b = 0; b < numBlocks; ++b) seq->add(block());     // every repeat reads the same lines
    out = seq;
  } else {
    out = block();
  }
  *parsed = taken;
  return out;
}

}  // namespace

std::shared_ptr<fl::Sequential> buildSequentialModule(const std::vector<std::string>& lines, int64_t nFeatures,
                                                      int64_t nClasses) {
  std::vector<std::string> layers;
  for (const std::string& raw : lines) {
    std::string l = trim(raw);
    replaceAll(l, "NFEAT", std::to_string(nFeatures));
    replaceAll(l, "NLABEL", std::to_string(nClasses));
    if (l.empty() || l[0] == '#') continue;   // blank lines and comments
    layers.push_back(l);
  }
  auto net = std::make_shared<fl::Sequential>();
  for (size_t i = 0; i < layers.size();) {
    size_t parsed = 0;
    net->add(parseLines(layers, i, &parsed));
    i += parsed + 1;
  }
  return net;
}

std::shared_ptr<fl::Sequential> buildSequentialModule(const std::string& archfile, int64_t nFeatures,
                                                      int64_t nClasses) {
  std::ifstream in(archfile);
  if (!in) throw std::runtime_error("fl::pkg::runtime::buildSequentialModule given invalid arch filepath");
  std::vector<std::string> lines;
  for (std::string s; std::getline(in, s);) lines.push_back(s);
  return buildSequentialModule(lines, nFeatures, nClasses);
}

}  // namespace runtime
}  // namespace pkg
}  // namespace fl
