// Batch readers of the benchmark applications (include/cavs/apps/readers.h): the parse-tree
// reader of apps/paper/tree-lstm-cavs.cc:30-103 and the token-stream loader of
// apps/paper/seq-lstm-cavs-varLength.cc:27-66, with their CHECKs turned into error returns.
#include "cavs/apps/readers.h"

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <fstream>
#include <sstream>
#include <string>
#include <vector>

namespace {

thread_local std::string g_error;

int fail(const char *fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  std::vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_error = buf;
  return -1;
}

// blank-separated integers of one line (reading stops at the first token that is not one,
// as `stream >> int` does)
std::vector<int> ints_of(const std::string &line) {
  std::vector<int> v;
  std::stringstream ss(line);
  int x;
  while (ss >> x) v.push_back(x);
  return v;
}

struct TreeReader {
  std::ifstream input, label, graph;
  void rewind() {
    for (std::ifstream *f : {&input, &label, &graph}) {
      f->clear();
      f->seekg(0, std::ios::beg);
    }
  }
};

struct PtbReader {
  int batch = 0, max_length = 0;
  std::vector<std::vector<float>> input, label;
  std::vector<std::vector<int>> graph;
};

}  // namespace

extern "C" {

const char *cavs_reader_last_error(void) { return g_error.c_str(); }

int cavs_tree_reader_open(const char *input_path, const char *label_path, const char *graph_path,
                          void **reader) {
  if (!input_path || !label_path || !graph_path || !reader) return fail("cavs_tree_reader_open: null argument");
  auto *r = new TreeReader;
  r->input.open(input_path);
  r->label.open(label_path);
  r->graph.open(graph_path);
  const char *bad = !r->input ? input_path : !r->label ? label_path : !r->graph ? graph_path : nullptr;
  if (bad) {
    delete r;
    return fail("cavs_tree_reader_open: cannot open %s", bad);
  }
  *reader = r;
  return 0;
}

int cavs_tree_reader_next(void *reader, int batch, int max_vertices, int max_words, int pack_inputs,
                          int *graph, float *input, float *label) {
  auto *r = static_cast<TreeReader *>(reader);
  if (!r || !graph || !input || !label) return fail("cavs_tree_reader_next: null argument");
  if (batch <= 0 || max_vertices <= 0 || max_words <= 0)
    return fail("cavs_tree_reader_next: bad sizes batch=%d max_vertices=%d max_words=%d", batch, max_vertices, max_words);
  const size_t total = (size_t)batch * max_vertices;
  std::fill(input, input + total, 0.f);
  std::fill(label, label + total, -1.f);
  std::fill(graph, graph + total, -1);
  int i = 0, label_length = 0, vertices = 0, rewinds_without_sample = 0;
  while (i < batch) {
    if (r->input.eof()) {  // the previous read ran into the end: start over
      if (++rewinds_without_sample > 1) return fail("cavs_tree_reader_next: the input file holds no sample");
      r->rewind();
    }
    std::string input_str, label_str, graph_str;
    std::getline(r->input, input_str);
    if (input_str.empty()) continue;
    rewinds_without_sample = 0;
    std::getline(r->label, label_str);
    std::getline(r->graph, graph_str);
    const std::vector<int> parents = ints_of(graph_str), words = ints_of(input_str), labels = ints_of(label_str);
    if (parents.empty() || parents.back() - 1 != -1)
      return fail("cavs_tree_reader_next: sample %d: the last vertex must be the root (parent 0)", i);
    if ((int)parents.size() > max_vertices)
      return fail("cavs_tree_reader_next: sample %d has %zu vertices, limit %d", i, parents.size(), max_vertices);
    if ((int)words.size() > max_words || (int)words.size() > max_vertices)
      return fail("cavs_tree_reader_next: sample %d has %zu words, limit %d", i, words.size(), std::min(max_words, max_vertices));
    if ((int)labels.size() > max_vertices || (size_t)label_length + labels.size() > total)
      return fail("cavs_tree_reader_next: sample %d has %zu labels, limit %d", i, labels.size(), max_vertices);
    for (size_t j = 0; j < parents.size(); j++) graph[(size_t)i * max_vertices + j] = parents[j] - 1;
    float *dst = pack_inputs ? input + vertices : input + (size_t)i * max_vertices;
    for (size_t j = 0; j < words.size(); j++) dst[j] = (float)words[j];
    for (size_t j = 0; j < labels.size(); j++) label[label_length + j] = (float)labels[j];
    label_length += (int)labels.size();
    vertices += (int)parents.size();
    i++;
  }
  return 0;
}

int cavs_tree_reader_close(void *reader) {
  delete static_cast<TreeReader *>(reader);
  return 0;
}

int cavs_ptb_reader_load(const char *path, int batch, int max_length, void **reader, int *n_batches) {
  if (!path || !reader || !n_batches) return fail("cavs_ptb_reader_load: null argument");
  if (batch <= 0 || max_length <= 0) return fail("cavs_ptb_reader_load: bad sizes batch=%d max_length=%d", batch, max_length);
  std::ifstream file(path);
  if (!file) return fail("cavs_ptb_reader_load: cannot open %s", path);
  auto r = new PtbReader;
  r->batch = batch;
  r->max_length = max_length;
  const size_t total = (size_t)batch * max_length;
  std::string s;
  bool end = false;
  long line_no = 0;
  while (!end) {
    std::vector<float> input_line(total, -1.f), label_line(total, -1.f);
    std::vector<int> graph_line(total, -1);
    size_t outer = 0;
    for (int sample = 0; sample < batch; sample++) {
      if (!std::getline(file, s)) {
        end = true;  // an incomplete batch is dropped
        break;
      }
      line_no++;
      std::stringstream ss(s);
      float tok = 0;
      int len = 0;
      while (ss >> tok) {
        if (len == max_length) {
          delete r;
          return fail("cavs_ptb_reader_load: line %ld has more than %d tokens", line_no, max_length);
        }
        input_line[outer + len] = tok;
        len++;
      }
      for (int j = 0; j + 1 < len; j++) {
        label_line[outer + j] = input_line[outer + j + 1];
        graph_line[(size_t)sample * max_length + j] = j + 1;
      }
      outer += len;
    }
    if (end) break;
    r->input.push_back(std::move(input_line));
    r->label.push_back(std::move(label_line));
    r->graph.push_back(std::move(graph_line));
  }
  *reader = r;
  *n_batches = (int)r->input.size();
  return 0;
}

int cavs_ptb_reader_batch(void *reader, int k, int *graph, float *input, float *label) {
  auto *r = static_cast<PtbReader *>(reader);
  if (!r || !graph || !input || !label) return fail("cavs_ptb_reader_batch: null argument");
  if (k < 0 || k >= (int)r->input.size()) return fail("cavs_ptb_reader_batch: batch %d of %zu", k, r->input.size());
  std::copy(r->input[k].begin(), r->input[k].end(), input);
  std::copy(r->label[k].begin(), r->label[k].end(), label);
  std::copy(r->graph[k].begin(), r->graph[k].end(), graph);
  return 0;
}

int cavs_ptb_reader_close(void *reader) {
  delete static_cast<PtbReader *>(reader);
  return 0;
}

}  // extern "C"
