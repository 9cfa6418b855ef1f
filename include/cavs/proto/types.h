// Plain-C++ restatement of the reference's protobuf enums (cavs/proto/types.proto,
// devices.proto, opt.proto): this toolchain has no protobuf.
#ifndef CAVS_PROTO_TYPES_H_
#define CAVS_PROTO_TYPES_H_

enum DataType { DT_FLOAT = 0, DT_DOUBLE = 1, DT_INT32 = 2 };
enum DeviceType { CPU = 0, GPU = 1 };
// cavs/proto/opt.proto:3-8
enum OptLevel { OPT_NONE = 0, OPT_FUSION = 1, OPT_BATCHING = 2, OPT_STREAMMING = 4 };

#endif
