// Host-side helpers shared between the device API and the file/codec code.
#pragma once
#include <stdint.h>

namespace l2j_host {
// Cache-file stem of a quantized tensor (J/TransformerWeights.java:54-111), or "" for the fp32 ones.
const char *tensor_stem(int tensor);
}  // namespace l2j_host

extern "C" void l2j_set_error_(const char *msg);
