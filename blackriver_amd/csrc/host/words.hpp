// Native words that expose the tensor operators to the word machine.
#pragma once

#include "vm.hpp"

namespace br {

// Registers the io.* and op.* words (same names and stack effects as the
// reference's load_nn_words, blackriver/nn.cpp:339-371) plus the extension
// word op.gemm_precision.
void load_nn_words(Enviroment& env);

}  // namespace br
