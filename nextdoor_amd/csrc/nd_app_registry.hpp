// How an application gets into the library's registry.
//
// The reference builds one binary per application: the application's source includes the
// engine (nextdoor.cu) and instantiates it on <SampleType, App> (src/apps/*/main.cu:1-21,
// src/tests/testBase.h:14-24).  Here the engine is instantiated the same way - in whatever
// translation unit names the pair, compiled by hipcc - and handed to libnextdoor_amd.so under a
// name with nd_register_app (include/nextdoor_amd.h); from then on the C ABI, the C++ host API
// and the Python mirror reach it like the applications compiled into the library.
//
//   #include "nd_app_registry.hpp"
//   struct MyApp { ... steps(), stepSize(), next(), ... };       // the App contract
//   ND_REGISTER_APP("MyApp", MySample, MyApp)                    // at namespace scope
//
// builds into a shared object of its own (hipcc -shared, linked against libnextdoor_amd.so);
// loading it (dlopen, a link dependency, ctypes.CDLL) registers the application.
#pragma once

#include <stdio.h>

#include <type_traits>

#include "../../include/nextdoor_amd.h"
#include "nd_engine.hpp"
#include "nd_layer_engine.hpp"
#include "nd_sharded_engine.hpp"
#include "nd_subgraph_engine.hpp"

namespace nd {

// Which engine serves an application:
//   kCollectiveEngine  samplingType() == CollectiveNeighborhood: the app carries
//                      kNeighborhoodForm (nd_apps_layer.hpp), or ND_COLLECTIVE_APP(App) declares a
//                      reference-style app whose next() gets no neighbourhood (the literal
//                      FastGCN / LADIES apps of the reference)
//   kEdgeListEngine    outputFormat() == AdjacencyMatrix on per-transit sampling, next() handing
//                      edges to sample->emit (the app carries kListsEdges)
//   kTransitEngine     everything else
enum EngineKind { kTransitEngine = 0, kCollectiveEngine = 1, kEdgeListEngine = 2 };

template <class App>
struct declared_collective { static constexpr bool value = false; };
template <class App, class = void>
struct app_engine_kind {
  static constexpr EngineKind value = declared_collective<App>::value ? kCollectiveEngine : kTransitEngine;
};
template <class App>
struct app_engine_kind<App, decltype((void)App::kNeighborhoodForm)> { static constexpr EngineKind value = kCollectiveEngine; };
template <class App>
struct app_engine_kind<App, decltype((void)App::kListsEdges)> { static constexpr EngineKind value = kEdgeListEngine; };

template <class SampleType, class App>
void* make_app_engine(const char* name) {
  EngineBase* engine;
  if constexpr (app_engine_kind<App>::value == kCollectiveEngine) engine = new LayerEngine<SampleType, App>(name);
  else if constexpr (app_engine_kind<App>::value == kEdgeListEngine) engine = new SubgraphEngine<SampleType, App>(name);
  else engine = new ShardedEngine<SampleType, App>(name);
  return engine;
}

// What nd_register_app compares: the hand-raised ND_ENGINE_ABI and the sizes of the structs a
// shared object of apps and the library both lay out (the engine's base class, the kernel
// parameters, the per-step bookkeeping).
constexpr int engine_abi() {
  return ND_ENGINE_ABI * 65536 + (int)((sizeof(EngineBase) + sizeof(StepParams) + sizeof(RunsMeta) + sizeof(PhaseTimes)) % 65536);
}

// Registers <SampleType, App> under `name` when the object is constructed (a namespace-scope
// object: when the shared object that holds it is loaded).  A refusal (name taken, other engine
// layout) is reported on stderr: nobody looks at a static object's members.
template <class SampleType, class App>
struct AppRegistration {
  explicit AppRegistration(const char* name) {
    rc = nd_register_app(name, &make_app_engine<SampleType, App>, engine_abi());
    if (rc != 0) fprintf(stderr, "nextdoor: app '%s' was not registered: %s\n", name, nd_last_error());
  }
  int rc;
};

}  // namespace nd

// At global scope, before ND_REGISTER_APP: App samples from the collective neighbourhood.
#define ND_COLLECTIVE_APP(...)                                 \
  namespace nd {                                               \
  template <>                                                  \
  struct declared_collective<__VA_ARGS__> {                    \
    static constexpr bool value = true;                        \
  };                                                           \
  }

#define ND_REGISTER_CONCAT2(a, b) a##b
#define ND_REGISTER_CONCAT(a, b) ND_REGISTER_CONCAT2(a, b)
#define ND_REGISTER_APP(name, SampleType, ...) \
  static nd::AppRegistration<SampleType, __VA_ARGS__> ND_REGISTER_CONCAT(nd_app_registration_, __LINE__)(name);
