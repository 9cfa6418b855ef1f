// Same include path as the reference's generated header so that applications compile
// unchanged; the content is a plain enum (cavs/proto/opt.proto:3-8).
#ifndef CAVS_PROTO_OPT_PB_H_
#define CAVS_PROTO_OPT_PB_H_
#include "cavs/proto/types.h"
#endif
