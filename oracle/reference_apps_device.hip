// TEST INFRASTRUCTURE ONLY.  The reference's own application sources, compiled by hipcc from
// where they lie under the reference tree (REFERENCE_ROOT, given by oracle/Makefile; nothing
// is copied into this repository) against the App contract header, instantiated on this
// repository's engine and registered with the library under "Reference..." names: the
// applications of src/apps dropped in unchanged (khop, randomwalks, fastgcn, ladies, layer,
// multiRW).  tests/test_gpu_reference_apps.py loads the
// shared object and compares what the engine samples with them on the GPU with the oracle.
//
// Not here: src/apps/mvs/mvsSampling.cu and src/apps/clustergcn/clusterGCNSampling.cu.  Their
// next() appends to lists in global storage through pointers kept in the sample state
// (sample->adjacencyMatrixRow[::atomicAdd(&sample->adjacencyMatrixLen, 1) + ...]) that the
// reference's main() allocates with cudaMalloc and sizes by host arithmetic, and ClusterGCN's
// stepTransits reserves room with an atomic on a global counter: text that cannot run without
// the reference's own allocation code around it, and whose output order depends on the
// schedule.  The library's MVS / ClusterGCN (nd_apps_subgraph.hpp) restate them on sample->emit.
#define ND_NO_REFERENCE_APP_NAMES  // the reference's FastGCNSample / FastGCNSamplingApp come from its own source
#include "../nextdoor_amd/csrc/nd_app_registry.hpp"

#include REFERENCE_KHOP
#include REFERENCE_RANDOM_WALKS
#undef VERTICES_PER_SAMPLE  // each app source sets its own
#include REFERENCE_FASTGCN
#include REFERENCE_LADIES  // the same four sizes again, with the same values
#undef VERTICES_PER_SAMPLE
#include REFERENCE_LAYER
#include REFERENCE_MULTIRW

ND_COLLECTIVE_APP(FastGCNSamplingApp)
ND_COLLECTIVE_APP(ImportanceSampleApp)

ND_REGISTER_APP("ReferenceKHop", KHopSample, KHopApp)
ND_REGISTER_APP("ReferenceDeepWalk", DummySample, DeepWalkApp)
ND_REGISTER_APP("ReferencePPR", DummySample, PPRApp)
ND_REGISTER_APP("ReferenceNode2Vec", Node2VecSample, Node2VecApp)
ND_REGISTER_APP("ReferenceFastGCN", FastGCNSample, FastGCNSamplingApp)
ND_REGISTER_APP("ReferenceLADIES", ImportanceSample, ImportanceSampleApp)
ND_REGISTER_APP("ReferenceLayer", LayerSample, LayerSamplingApp)
ND_REGISTER_APP("ReferenceMultiRW", MultiRWSample, MultiRWApp)
