// Description of a vertex function of the general shape (one stage of products; several stages are
// a chain of such descriptions, see CellSpec::next)
//
//   state' , ret = f( x*W , sum_t A_t * B_t , bias , states of the children )      (f elementwise)
//
// as the engine runs it on generated round kernels: which views of which parameters feed the
// products, which sums of children's state blocks are their left operands, how many values a vertex
// keeps for the backward pass, and the source of the kernels (the product loops written out for this
// function, the elementwise part f and its derivative generated from the operator graph).  Takes the
// place of the reference's kernel fusion for a whole vertex function
// (cavs/midend/runtime_compiler/parser.cc:73-139, code_generator.cc:104-185) with the products inside.
#ifndef CAVS_HOST_CELL_H_
#define CAVS_HOST_CELL_H_

#include <memory>
#include <string>
#include <vector>

namespace cavs {

struct CellParamRef {
  int param = -1;    // index into CellSpec::params
  long offset = 0;   // first element of the view inside that parameter
};

// Left operand of a product: the sum over the children in `mask` (bit k = child k) of block `block`
// of their state rows; a missing child contributes zero.
struct CellASrc {
  int mask = 0, block = 0;
};

// One accumulator of the round kernels: sum over its terms of  A[asrc] (1 x H)  *  B[brow .. brow + H) x [col .. col + H).
struct CellTerm {
  int asrc = 0;
  long brow = 0;
};
struct CellProduct {
  std::vector<CellTerm> terms;
  CellParamRef B;   // the view the rows and columns count from, row-major with leading dimension ldb
  int ldb = 0;
  long col = 0;
  int dcol = -1;    // block of the per-vertex gradient rows that holds d(this accumulator)
};

struct CellBias {
  CellParamRef ref;  // H values
  int dcol = -1;     // block of the gradient rows whose column sums are its gradient
  bool add = false;  // an earlier cell of the chain reads the same bias: this cell's share is added to that one's
};

struct CellParam {
  std::string name;  // engine parameter ("Emb" for the embedding table, else "P<i>")
  long size = 0;
};

struct CellSpec {
  int H = 0, K = 0, S = 0;      // block width, children per vertex, state blocks of the message it writes
  int SI = 0;                   // state blocks of the rows it gathers (the children's messages; = S for a function of one stage)
  int E = 0, V = 0, NX = 0;     // embedding width, vocabulary, blocks of x * W (0: F looks no vertex input up)
  int XD = 0;                   // H-wide blocks of the vertex input's row that F pulls and uses as they are
  CellParamRef W;               // [E, NX * H]
  int xw_lo = 0, xw_hi = 0;     // the blocks of x * W this cell reads: [xw_lo, xw_hi) (the gradient rows' other x * W blocks are zero)
  std::vector<CellParam> params;
  std::vector<CellASrc> asrc;
  std::vector<CellProduct> products;
  std::vector<CellBias> biases;
  int ND = 0;                   // blocks of a vertex's gradient row: d(x*W) blocks first, in order
  int NSV = 0;                  // blocks a vertex saves for the backward pass
  int waves = 0;                // wavefronts per workgroup of the round kernels (they split the k range)
  std::string source;           // the kernels (equal sources share a compiled module)
  // A vertex function of several stages -- a product whose left operand depends on another product
  // of the same vertex -- runs as a chain of such cells: every cell but the last writes, per vertex,
  // a row of intermediate blocks (the next stage's left operands and whatever later stages read of
  // this one), which the next cell gathers as the state of its one "child", the vertex itself.
  std::shared_ptr<CellSpec> next;
  bool has_ret = true;          // the last cell of a chain pushes the return value
  int terms() const {
    int n = 0;
    for (const CellProduct &p : products) n += (int)p.terms.size();
    return n;
  }
  // the distinct H x H weight blocks the terms read (a block may serve several terms)
  int blocks() const {
    std::vector<long> seen;  // (param, ldb, first element) triples
    for (const CellProduct &p : products)
      for (const CellTerm &t : p.terms) {
        const long key[3] = {p.B.param, p.ldb, p.B.offset + t.brow * p.ldb + p.col};
        bool found = false;
        for (size_t i = 0; i + 2 < seen.size() && !found; i += 3) found = seen[i] == key[0] && seen[i + 1] == key[1] && seen[i + 2] == key[2];
        if (!found) seen.insert(seen.end(), key, key + 3);
      }
    return (int)(seen.size() / 3);
  }
};

// Order of the 8-byte argument slots of the generated kernels (struct CellArgs in their source).
enum CellArg {
  CA_POOL = 0,   // float*  the rows this cell's state goes to [*, S*H]
  CA_CHILD,      // int*    pool rows of the children by slab row [K * N]
  CA_PAIR,       // int*    pool row a slab row's message goes to [N]
  CA_KIDS,       // int*    slab rows of the children by slab row [K * N]
  CA_T2J,        // int*    vertex id by slab row [N]
  CA_ROWS,       // int*    slab rows for the rows kernel (the vertices nobody sends a gradient to)
  CA_XW,         // float*  [N, NX*H]
  CA_SV,         // float*  [N, NSV*H]
  CA_ASRC,       // float*  [N, NA*H]
  CA_GO,         // float*  [N, H] by vertex id: the pushed value / its gradient
  CA_D,          // float*  [N, ND*H]
  CA_DS,         // float*  [N, SI*H] elementwise part of a vertex's message gradient by slab row; or, for
                 //         cell_bwd_gates / cell_bwd_pool, [K * n, SI*H] by row of the round and child
  CA_BT,         // float*  tile-major copies of the weight blocks: as they are, then transposed
  CA_COLSUM,     // float*  [ND*H] column sums of D
  CA_DPOOL,      // float*  gradient of the rows this cell's state goes to [*, S*H] (cell_bwd_gates reads it)
  CA_X,          // float*  the vertex input by vertex id [*, XD*H]
  CA_POOL_IN,    // float*  the rows this cell gathers its children's states from [*, SI*H] (a function of one stage: CA_POOL)
  CA_DPOOL_IN,   // float*  gradient of those rows (cell_bwd_pool writes it; a function of one stage: CA_DPOOL)
  // the cell whose rows this one gathers (itself for a function of one stage; in a chain the cell
  // before, and for the first cell the last): cell_bwd runs the elementwise part of its backward
  // function on the message gradients its products complete
  CA_FT_SV,      // float*  that cell's kept values
  CA_FT_D,       // float*  its gradient rows
  CA_FT_DS,      // float*  elementwise part of the gradients of the rows it gathers, by slab row
  CA_FT_POOL_IN, // float*  the rows it gathers
  CA_FT_CHILD,   // int*    rows of those by slab row
  CA_FT_KIDS,    // int*    slab rows of its children by slab row
  CA_OFF,        // long    first slab row of the round
  CA_N,          // long    rows
  CA_PARAM0,     // float*  parameters, then their gradients, in CellSpec::params order
  CA_MAX_PARAMS = 8,
  CA_SLOTS = CA_PARAM0 + 2 * CA_MAX_PARAMS
};

// kernels of a compiled cell, in the order cavs_cell_compile looks them up
enum CellKernel { CK_FWD = 0, CK_LEAVES, CK_BWD, CK_BWD_ROWS, CK_PACK, CK_BIAS, CK_BWD_GATES, CK_BWD_POOL, CK_COUNT };

}  // namespace cavs
#endif
