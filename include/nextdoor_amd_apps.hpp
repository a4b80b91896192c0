// The applications compiled into libnextdoor_amd.so, as types: the reference's app structs
// under their own names (UniformRandomWalkApp, DeepWalkApp, PPRApp, Node2VecApp, KHopApp,
// LayerSamplingApp, MultiRWApp, MVSSamplingApp, SubGraphSamplingAppI, FastGCNSamplingApp,
// ImportanceSampleApp and their SampleTypes; src/apps/*, example/uniformRandWalk.cu), each with
// the registry name the template host API (libNextDoor_amd.hpp) looks it up by.  Takes the place
// of the reference's `#include "../apps/khop/khop.cu"` in a caller's source
// (src/tests/singleGPU/khop.cu:1-3).  Compiles in a host-only translation unit as well.
#ifndef NEXTDOOR_AMD_APPS_HPP
#define NEXTDOOR_AMD_APPS_HPP

#include "../nextdoor_amd/csrc/nd_apps_khop.hpp"
#include "../nextdoor_amd/csrc/nd_apps_multirw.hpp"
#include "../nextdoor_amd/csrc/nd_apps_subgraph.hpp"
#include "../nextdoor_amd/csrc/nd_apps_walks.hpp"
#if defined(__HIPCC__)
#include "../nextdoor_amd/csrc/nd_apps_layer.hpp"  // its importance forms name device-side types of the layer engine
#endif

#endif
