// Builds a Sequential from wav2letter-style architecture lines, one module per line, as
// flashlight/pkg/runtime/common/SequentialBuilder.cpp:28-67 (file reading, NFEAT / NLABEL
// substitution, blank lines and '#' comments) and :98-640 (the line grammar) do.  The
// lines whose modules exist in Modules.h build exactly what the reference builds:
//   V d0 d1 ..                      View
//   C|C1 in out wx sx [px [dx]]     Conv2D(in, out, wx, 1, sx, 1, px, 0, dx, 1)   (px -1 = SAME)
//   C2 in out wx wy sx sy [px [py [dx [dy]]]]
//   L in out [0 = no bias]          Linear
//   BN feat axis [axis ..]          BatchNorm(axes, feat)
//   LN axis [axis ..]               LayerNorm(axes)
//   M|A wx wy sx sy [px [py]]       Pool2D (MAX | AVG_INCLUDE_PADDING)
//   R                               ReLU
//   LSM dim                         LogSoftmax
//   RNN|GRU|LSTM in out [layers [bidirectional [dropout]]]
// A well-formed line for a module this backend does not have (RO, PD, TR, CFR, POSEMB,
// SINPOSEMB, TDS, AC, E, ADAPTIVEE, WN, DO, ELU, R6, PR, LG, HT, T, GLU, SH, RES, SAUG,
// PC) throws std::invalid_argument naming the module; anything else throws
// "Failed parsing - <line>" like the reference.
#pragma once

#include <cstdint>
#include <memory>
#include <string>
#include <vector>

#include "Modules.h"

namespace fl {
namespace pkg {
namespace runtime {

std::shared_ptr<fl::Sequential> buildSequentialModule(const std::string& archfile, int64_t nFeatures,
                                                      int64_t nClasses);
// the same from lines already in memory
std::shared_ptr<fl::Sequential> buildSequentialModule(const std::vector<std::string>& lines, int64_t nFeatures,
                                                      int64_t nClasses);

}  // namespace runtime
}  // namespace pkg
}  // namespace fl
