// Host-side topological ordering of a CSR graph given as successor lists, with
// the reference's rule for graphs that are not acyclic
// (topo_sort, src/cpp/src/schedule.cu:71-128).  Sequential queue algorithm on
// host memory: the reference runs it on CPU tensors and so does this.
//
//   1. every node whose counter is 0 enters a FIFO queue in id order;
//   2. a dequeued node is emitted and the counters of its successors drop by
//      one; a counter reaching exactly 0 enqueues its node;
//   3. when the queue runs dry before all nodes are out: every node whose
//      counter is 1 is enqueued (counter := 0) and so is the FIRST node with the
//      smallest counter above 1 among the nodes scanned before it changed
//      (the scan keeps a running minimum, as the reference does); if nothing
//      was enqueued the walk stops.
// Returns the number of nodes emitted; entries past it are left untouched.
#include "cxg_common.hpp"

#include <queue>
#include <vector>

extern "C" {

int64_t cxg_topo_sort_host_i64(const int64_t* ptr, const int64_t* idx, const int64_t* degree,
                               int64_t n_nodes, int64_t* order) {
  if (n_nodes < 0 || (n_nodes > 0 && (!ptr || !degree || !order))) {
    return cxg::set_error(CXG_ERR_ARG, "cxg_topo_sort_host_i64: bad arguments");
  }
  std::vector<int64_t> deg(degree, degree + n_nodes);
  std::queue<int64_t> q;
  for (int64_t i = 0; i < n_nodes; ++i)
    if (deg[i] == 0) q.push(i);
  int64_t cnt = 0;
  while (cnt < n_nodes) {
    while (!q.empty()) {
      const int64_t cur = q.front();
      q.pop();
      order[cnt++] = cur;
      for (int64_t k = ptr[cur]; k < ptr[cur + 1]; ++k) {
        const int64_t next = idx[k];
        if (--deg[next] == 0) q.push(next);
      }
    }
    int64_t min_deg = n_nodes, pick = -1;
    for (int64_t i = 0; i < n_nodes; ++i) {
      if (deg[i] < min_deg && deg[i] > 1) {
        min_deg = deg[i];
        pick = i;
      } else if (deg[i] == 1) {
        deg[i] = 0;
        q.push(i);
      }
    }
    if (pick != -1) {
      q.push(pick);
      deg[pick] = 0;
    } else if (q.empty()) {
      break;
    }
  }
  return cnt;
}

}  // extern "C"
