// Host-side mirror of CNet's public C++ API over the MI355X device library (include/cnet_hip.h).
//
// Same class names, constructor arguments, method names and error behaviour as upstream CNet for the dense complex
// path (upstream gpu/gpu_func.h:41-1113, impl/cfunc.h, impl/cnet.h, impl/vars.h, impl/batch.h and the layer
// headers), so a program written against upstream -- net.add(new Linear(...), {x, w}); allocateOnGpu(B);
// gpuForward(inp, out, batch); getLoss(...); gpuBackward(); gpuUpdateInputs(lr / B) -- compiles against this header.
// What is underneath is different by design:
//   * no per-sample graph clones: one node = one set of batched device planes [rows x len]; parameter nodes
//     (every CInput that is not the data input, and the embedding table) are stored ONCE (rows = 1);
//   * a producer owns its output planes and each consumer reads them in place (no copies into consumer blocks; fan-out
//     costs nothing); every consumer slot owns its four gradient planes;
//   * every layer step is a call into the C ABI (batched GEMMs / fused elementwise / wavefront reductions) queued on
//     one stream; nothing synchronises until a result is read back.
// There is NO CPU execution path here: forward()/backward()/updateInputs() of the per-sample API also run on the
// device (batch of one), and every method fails loudly (std::runtime_error) when the device layer reports an error.
//
// Host views: net[uid]->input() is the per-sample six-plane block of upstream (impl/vars.h:40-46).  The batched calls
// leave results on the device; CNet::fetch(node, batch_index) fills a node's host view for one sample
// (upstream: testDataFromGpu / printMappingFromGpu copy a mapping back, gpu/gpu_func.h:700-862).
#ifndef CNET_AMD_HOST_CNET_HPP_
#define CNET_AMD_HOST_CNET_HPP_

#include <algorithm>
#include <cassert>
#include <cmath>
#include <complex>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <ctime>
#include <initializer_list>
#include <iomanip>
#include <iostream>
#include <map>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "cnet_hip.h"

#include "vars.hpp"
#include "batches.hpp"
#include "functions.hpp"
#include "net.hpp"
#include "model_saver.hpp"

#endif  // CNET_AMD_HOST_CNET_HPP_
