// ONNX files for the CNN forward path, in C++: the reference's entry points
//   import_net_from_onnx_file / _pointer / _string   src/serialization/onnx/net/eddl_onnx_import.cpp:19-93
//   save_net_to_onnx_file, serialize_net_to_onnx_string  src/serialization/onnx/net/eddl_onnx_export.cpp:17-78
// with the behaviour of its importer and exporter for the layers of this path
// (import_helpers.cpp:210-243,529-710, export_helpers.cpp:8-120, layers/*_onnx.cpp).  The reference
// parses with protobuf-generated classes; here the messages involved are read and written straight
// from the protobuf wire format, so the host layer keeps building with g++ alone.
#pragma once
#include <cstddef>

#include "eddl_hip_net.h"

namespace eddl_hip {

// input_shape: without the batch; empty = the shape the file states.  The net comes back on the
// host, not built: call eddl::build(net, CS_HIP({1}), false) to keep the imported parameters.
Net *import_net_from_onnx_file(const string &path, const vector<int> &input_shape = {}, int mem = 0);
Net *import_net_from_onnx_pointer(const void *serialized_model, size_t size, int mem = 0);
Net *import_net_from_onnx_string(const string *model_string, int mem = 0);

void save_net_to_onnx_file(Net *net, const string &path);
string serialize_net_to_onnx_string(Net *net);

}  // namespace eddl_hip
