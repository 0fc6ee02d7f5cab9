// C wrappers around the reference's own Partition / TwistedHyperCube translation units, so the
// tests can call the real reference code through ctypes.  TEST INFRASTRUCTURE ONLY.
// This file is compiled together with Partition.cc and TwistedHyperCube.cc taken from the
// reference checkout where it lies (see Makefile target `ref`); only the resulting shared
// object, oracle/_ref/libref_partition.so, is used.  Nothing from the reference is copied.
#include "Partition.h"         // reference header, found through -I$(REFERENCE)
#include "TwistedHyperCube.h"  // reference header

extern "C" {

void ref_set_nsockets(int n) { nsockets = n; }

int ref_get_work_per_socket(int work) { return get_work_per_socket(work); }

// Partition.cc:30-48
void ref_get_partition(int work, int sid, int T, int t, int* out2) {
  std::pair<int, int> p = get_partition(work, sid, T, t);
  out2[0] = p.first;
  out2[1] = p.second;
}

// Partition.cc:75-166
void ref_get_intra_socket_2dpartition(int m, int n, double ar, int m_align, int T, int t,
                                      int* out4) {
  get_intra_socket_2dpartition(&out4[0], &out4[1], &out4[2], &out4[3], m, n, ar, m_align != 0, T,
                               t);
}

// Partition.cc:193-222
void ref_get_2dpartition(int m, int n, double ar, int m_align, int sid, int T, int t, int* out4) {
  get_2dpartition(&out4[0], &out4[1], &out4[2], &out4[3], m, n, ar, m_align != 0, sid, T, t);
}

// TwistedHyperCube.cc:9-52 (twisted == 0) and :60-123 (twisted != 0); what = 0 Peer, 1 Recv, 2 Send
int ref_hypercube(int twisted, int num_nodes, int shift, int what, int id, int dim) {
  if (twisted) {
    TwistedHyperCube c(num_nodes, shift);
    return what == 0 ? c.Peer(id, dim) : what == 1 ? c.RecvLocation(id, dim) : c.SendLocation(id, dim);
  }
  HyperCube c(num_nodes, shift);
  return what == 0 ? c.Peer(id, dim) : what == 1 ? c.RecvLocation(id, dim) : c.SendLocation(id, dim);
}

}  // extern "C"
