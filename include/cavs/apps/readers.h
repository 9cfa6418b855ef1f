/* Batch readers of the benchmark applications: the text formats either side of the
 * vertex-function path.
 *
 *  - parse-tree corpora (SST): three files with one sample per line of blank-separated
 *    integers -- word ids of the leaves, one label per vertex, and the parent of every
 *    vertex counted from 1 with 0 for the root, which must come last.  Replaces
 *    `class Reader` of apps/paper/tree-lstm-cavs.cc:30-103 (the files are the ones
 *    apps/lstm/preprocess.py:50-76 writes next to labels.txt and parents.txt).
 *  - token streams (PTB): one sentence of token ids per line; labels are the next token,
 *    the graph is the chain j -> j+1.  Replaces load() of
 *    apps/paper/seq-lstm-cavs-varLength.cc:27-66.
 *
 * Every function returns 0, or a negative code after storing a message for
 * cavs_reader_last_error(); nothing aborts.  Host memory only: no device is touched.
 */
#ifndef CAVS_APPS_READERS_H_
#define CAVS_APPS_READERS_H_

#ifdef __cplusplus
extern "C" {
#endif

const char *cavs_reader_last_error(void);

/* ---- parse trees (apps/paper/tree-lstm-cavs.cc:30-103) ---- */
int cavs_tree_reader_open(const char *input_path, const char *label_path, const char *graph_path,
                          void **reader);
/* Fills one batch.  graph[batch*max_vertices] = -1, then row i = parents of sample i minus 1
 * (-1 = root, last entry of the sample); label[batch*max_vertices] = -1, then the labels of all
 * samples packed back to back in vertex order; input[batch*max_vertices] = 0, then the word ids.
 * pack_inputs = 0 lays the word ids of sample i out at input[i*max_vertices ...] exactly as the
 * reference does (tree-lstm-cavs.cc:62); pack_inputs = 1 puts the ids of sample i at the global
 * vertex ids of its vertices (the first vertex of sample i is the sum of the vertex counts before
 * it), which is the order Pull reads them in (cavs/backend/op_impl_graphop.cu:208-258).
 * Empty lines are skipped; at the end of the files reading starts over from the beginning.
 * A sample with more than max_vertices vertices or more than max_words words is an error. */
int cavs_tree_reader_next(void *reader, int batch, int max_vertices, int max_words, int pack_inputs,
                          int *graph, float *input, float *label);
int cavs_tree_reader_close(void *reader);

/* ---- token streams (apps/paper/seq-lstm-cavs-varLength.cc:27-66) ---- */
/* Reads the whole file into batches of `batch` sentences; a last incomplete batch is dropped.
 * A sentence longer than max_length tokens is an error. */
int cavs_ptb_reader_load(const char *path, int batch, int max_length, void **reader, int *n_batches);
/* Batch k: input[batch*max_length] and label[batch*max_length] start at -1; the tokens of all
 * sentences are packed back to back into input, label holds the next token of the same sentence
 * at the same offsets (one fewer than the tokens, the rest stays -1);
 * graph[batch*max_length] = -1 with graph[s*max_length + j] = j + 1 for j < len(s) - 1. */
int cavs_ptb_reader_batch(void *reader, int k, int *graph, float *input, float *label);
int cavs_ptb_reader_close(void *reader);

#ifdef __cplusplus
}
#endif
#endif
