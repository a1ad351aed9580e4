// The statement log: what the frontend records (array creations, element-wise operations,
// assignments into regions, reductions and products, handles going away), one small record per
// operation, and the planner that turns a stretch of it into DAG nodes: which operations become one
// fused group, which results never need to exist as arrays, which deletions have nothing to delete.
// Upstream does this grouping on the Python side, in charmtyles (a dependency that is not part of
// the charmnumeric tree), and ships the finished DAG (src/dag_group_receive.cpp:190-192); here the
// frontend ships the raw log and the grouping runs natively, off the recording thread.
#pragma once
#include "decomp.h"

#include <cstdint>
#include <set>
#include <vector>

namespace cnh {
namespace stmtlog {

enum Kind { kCreate = 1, kOp = 2, kSet = 3, kNonfusible = 4, kDelete = 5 };

struct Ref {
    bool is_array = false;
    double scalar = 0.0;
    int32_t name = 0, base_ndims = 0, dtype = 0, broadcast = 0;
    bool has_region = false;
    cnh_region region;          // relative to the base array, when has_region
};

struct Instr {
    int32_t kind = 0, name = 0, opcode = 0, dtype = 0;
    int32_t ndims = 0, shape[3] = {0, 0, 0};
    int32_t n_operands = 0;
    Ref operands[2];
    int32_t target_ndims = 0;   // kSet: rank of the array assigned into
    cnh_region region;          // kSet: the region assigned, relative to that array
};

// Appends the records of `log` to `out`. 0, or < 0 with the error text set.
int parse(const char* log, int64_t size, std::vector<Instr>& out);

// Where an automatic flush stops: the number of leading instructions to plan now. A loop of the form
//     upd = f(u[...], ...)            (a result with a name of its own)
//     u[...] = g(u[...], upd)         (consumed by the next statement)
// leaves `upd` alive at every statement boundary, its handle going only when the name is bound
// again one iteration later; planning right there would turn it into a real array and split the
// statement in two. So the statements from the one that produced such a recent (within `window`
// instructions of the end), still undeleted result onwards stay behind.
size_t hold_back_cut(const std::vector<Instr>& batch, int window);

// Results produced in batch[0, cut) whose deletion waits in batch[cut, end) and which nothing there
// reads or assigns: the planner may treat them as already gone.
std::set<int32_t> dead_later(const std::vector<Instr>& batch, size_t cut);

// Plans batch[0, count) into DAG nodes appended to `out`, in execution order, ids from 0.
// `next_set_name` supplies the (otherwise unused) result names of SET_REGION roots. Names of
// `dead` that did not become arrays are added to `fused_away`.
void plan(const std::vector<Instr>& batch, size_t count, const std::set<int32_t>& dead,
          int32_t* next_set_name, std::vector<DagNode>& out, std::set<int32_t>* fused_away);

// The DAG message (format of include/cnexec.h) holding `nodes`.
std::vector<char> to_message(const std::vector<DagNode>& nodes);

} // namespace stmtlog
} // namespace cnh
