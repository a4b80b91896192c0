// TEST INFRASTRUCTURE ONLY.  The reference's own application sources, compiled by hipcc from
// where they lie under the reference tree (REFERENCE_ROOT, given by oracle/Makefile; nothing
// is copied into this repository) against the App contract header, instantiated on this
// repository's engine and registered with the library under "Reference..." names: the
// applications of src/apps dropped in unchanged.  tests/test_gpu_reference_apps.py loads the
// shared object and compares what the engine samples with them on the GPU with the oracle.
#define ND_NO_REFERENCE_APP_NAMES  // the reference's FastGCNSample / FastGCNSamplingApp come from its own source
#include "../nextdoor_amd/csrc/nd_app_registry.hpp"

#include REFERENCE_KHOP
#include REFERENCE_RANDOM_WALKS
#undef VERTICES_PER_SAMPLE  // each app source sets its own
#include REFERENCE_FASTGCN

ND_COLLECTIVE_APP(FastGCNSamplingApp)

ND_REGISTER_APP("ReferenceKHop", KHopSample, KHopApp)
ND_REGISTER_APP("ReferenceDeepWalk", DummySample, DeepWalkApp)
ND_REGISTER_APP("ReferencePPR", DummySample, PPRApp)
ND_REGISTER_APP("ReferenceNode2Vec", Node2VecSample, Node2VecApp)
ND_REGISTER_APP("ReferenceFastGCN", FastGCNSample, FastGCNSamplingApp)
