/*
 * Outer C API of the front end, same functions as the reference's
 * cavs/frontend/c_api.h:20-36.  Definitions cross as serialized bytes; the encoding is
 * this build's own (OpDef::SerializeToString), not protobuf.
 * Functions that the reference lets abort (CHECK) throw nothing across this boundary:
 * they print the message and abort like the reference, because the reference's
 * signatures have no error channel.  Extensions (no counterpart in the reference) are
 * marked.
 */
#ifndef CAVS_FRONTEND_C_API_H_
#define CAVS_FRONTEND_C_API_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum { C_FLOAT = 0, C_DOUBLE = 1, C_INT32 = 2 } C_Dtype;

typedef struct C_Session C_Session;
typedef struct C_Tensor C_Tensor;

C_Session *C_NewSession(const char *name, size_t name_len, int opt);
C_Tensor *C_NewTensor(const char *name, size_t name_len, const int *shape, int dims, C_Dtype dtype);
/* dim is allocated with malloc and owned by the caller (the reference does the same,
 * cavs/frontend/cxx/sym.cc:46) */
void C_AddOp(const void *def, size_t def_length, int **dim, size_t *dim_length);
void C_AddOptimizerOp(const void *def, size_t def_length);
void C_AddFunction(const void *def, size_t def_length, int **dim, size_t *dim_length);
void C_AddControlDependency(const void *def, size_t def_length);
void C_Run(C_Session *s, const char **c_output_names, C_Tensor **c_output_tensors, int noutputs,
           const char **c_input_names, C_Tensor *const *c_input_tensors, int ninputs);
void *C_TensorData(const C_Tensor *t);
size_t C_TensorSize(const C_Tensor *t);

/* ---- extensions ---- */
/* Drops the process-wide graph (the reference keeps one global main scope for the
 * life of the process); lets one process declare several programs one after another. */
void C_ResetGraph(void);
void C_DeleteSession(C_Session *s);
/* C_Run that reports a failure (non-zero, message in C_LastError) instead of aborting. */
int C_TryRun(C_Session *s, const char **c_output_names, C_Tensor **c_output_tensors, int noutputs,
             const char **c_input_names, C_Tensor *const *c_input_tensors, int ninputs);
void C_DeleteTensor(C_Tensor *t);
/* Overwrites a Variable with caller data instead of its filler (n = element count). */
int C_SetVariable(C_Session *s, const char *name, const float *data, size_t n);
/* Copies any tensor of the last run to host by edge name ("X" or "X_grad");
 * returns the element count, or the negative needed capacity, or 0 if unknown. */
long C_ReadTensor(C_Session *s, const char *name, float *out, size_t cap);
/* Whether the vertex function was lowered onto fused round kernels: 0 no (it runs op by op),
 * 1 onto the hand-written kernels of a recognised function, 2 onto kernels generated for it. */
int C_SessionUsesFusedPath(C_Session *s);
/* Number of kernels the OPT_FUSION pass generated for the programs compiled so far. */
int C_SessionGeneratedKernels(C_Session *s);
/* 0 forbids that lowering (op-by-op execution of F, for A/B tests); 1, the default, tries the
 * hand-written kernels first and generated ones next; 2 goes for generated kernels only; 3 does the
 * same and runs the backward rounds the way a batch whose message flow is no forest needs them
 * (two launches per round, message gradients through the gradient of the message pool). */
void C_SessionAllowFusedPath(C_Session *s, int allow);
void C_SessionSetPairing(C_Session *s, int pairing); /* CAVS_PAIR_* of cavs_session.h */
const char *C_LastError(void);
/* Text dump of the declared program: forward ops, the vertex function, and the backward
 * programs the autograd pass derived.  Returns the length needed (including the NUL). */
size_t C_DumpGraph(char *buf, size_t cap);
/* The kernels generated for the declared vertex function when it has the general shape (what = 1),
 * or its elementwise parts alone as host C++ (what = 0); a comment saying why not otherwise.  A
 * function of several stages is a chain of cells: what + 10 * s names cell s of it. */
size_t C_DumpCell(char *buf, size_t cap, int what);
/* The same programs after the OPT_FUSION pass, with the generated kernel sources. */
size_t C_DumpFusedGraph(char *buf, size_t cap);

#ifdef __cplusplus
}
#endif
#endif
