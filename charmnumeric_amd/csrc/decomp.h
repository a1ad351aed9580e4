// Decomposition planning for one DAG message: tile edge and offset of every array the message
// produces, as upstream's ArrayDAGGroup decides them before it expands partitions
// (src/decomposition_solver.hpp:94-1714, called from src/dag_group_receive.cpp:399).
#pragma once
#include "../../include/cnhip.h"

#include <cstdint>
#include <map>
#include <vector>

namespace cnh {

// One node of the DAG message: a flat AST whose last root is what the node does.
struct DagNode {
    int id = 0;
    int fusible = 0;
    std::vector<cnh_ast_node> nodes;
    std::vector<int32_t> roots;
};

// ArrayMetadata (src/backend.hpp:264-288): what the solver reads and writes per array.
struct DecompMeta {
    int ndims = 0;
    int32_t shape[3] = {0, 0, 0};
    int32_t offset[3] = {0, 0, 0};
    int tile = 0;
    bool final = false; // decided by an earlier message: never changed again
};

// Fills tile and offset of every entry that is not final, then marks all entries final.
// min_tile[r] is the smallest tile edge of rank r (1..3). Entries are visited in ascending name
// order and DAG nodes in the order listed; upstream walks hash maps, so where several choices tie
// (component root among several fixed arrays, the start of a component without any) its answer
// depends on the map's iteration order and only one of the tied answers is reproduced here.
void solve_decompositions(std::map<int, DecompMeta>& meta, const std::vector<DagNode>& dag, int odf,
                          int num_pes, const int min_tile[4]);

} // namespace cnh
