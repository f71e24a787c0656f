// CPU build of the allocator's bookkeeping (cl-waffe2_amd/csrc/wf2_pool.h) behind a
// small C interface that tests/test_pool_cpu.py drives.  Blocks are plain host
// allocations; test infrastructure only.
#include <cstdlib>
#include <vector>

#include "../../cl-waffe2_amd/csrc/wf2_pool.h"

using wf2::BlockPool;
using wf2::GraphBlocks;

extern "C" {
void* pool_new(int enabled) {
  BlockPool* p = new BlockPool();
  p->enabled = enabled != 0;
  return p;
}
void pool_delete(void* pool) {
  BlockPool* p = (BlockPool*)pool;
  std::vector<void*> release;
  p->drain_idle(&release);
  for (void* q : release) free(q);
  delete p;
}
void* graph_new() { return new GraphBlocks(); }
// like wf2hip_malloc_uninitialized: nullptr when a capture would have to allocate
void* pool_alloc(void* pool, unsigned long bytes, void* capture) {
  BlockPool* p = (BlockPool*)pool;
  const size_t cls = BlockPool::size_class(bytes);
  void* q = p->take(cls, (GraphBlocks*)capture);
  if (q || capture) return q;
  q = malloc(cls);
  p->adopt(q, cls);
  return q;
}
// 0 unknown pointer, 1 kept by the pool or a graph, 2 released
int pool_free(void* pool, void* ptr, void* capture) {
  BlockPool* p = (BlockPool*)pool;
  BlockPool::Outcome o = p->give_back(ptr, (GraphBlocks*)capture);
  if (o == BlockPool::kRelease) free(ptr);
  return (int)o;
}
// number of blocks released to the system
int graph_destroy(void* pool, void* graph) {
  std::vector<void*> release;
  ((BlockPool*)pool)->forget_graph((GraphBlocks*)graph, &release);
  for (void* q : release) free(q);
  delete (GraphBlocks*)graph;
  return (int)release.size();
}
unsigned long pool_idle_bytes(void* pool) { return ((BlockPool*)pool)->idle_bytes(); }
unsigned long pool_blocks_known(void* pool) { return ((BlockPool*)pool)->blocks_known(); }
unsigned long pool_owners_of(void* pool, void* ptr) { return ((BlockPool*)pool)->owners_of(ptr); }
unsigned long graph_held(void* graph) { return ((GraphBlocks*)graph)->held.size(); }
unsigned long pool_size_class(unsigned long bytes) { return BlockPool::size_class(bytes); }
}
