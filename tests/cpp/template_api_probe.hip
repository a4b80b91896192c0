// A caller written the way the reference's app binaries and tests are
// (src/apps/khop/main.cu:1-27, src/tests/testBase.h:14-24, example/uniformRandWalk.cu:95-122):
// the App struct, then appMain<SampleType, App>(argc, argv, checker).  Built by hipcc, as the
// reference's are by nvcc: the engine is instantiated for the caller's own App in this
// translation unit.  With "--registry-app" as the first argument it runs the testBase.h macro
// for an App that is compiled into the library instead.
#include <libNextDoor_amd.hpp>
#include <nextdoor_amd_apps.hpp>

// what next() leaves behind for the checker: the vertex the walk last stepped from, and how
// many times it stepped
struct CallerWalkSample {
  VertexID_t previous;
  int stepsTaken;
};

// the reference's example app (example/uniformRandWalk.cu:15-93) with walks of 6 steps
struct CallerWalkApp {
  __host__ __device__ int steps() { return 6; }
  __host__ __device__ int stepSize(int k) { return 1; }

  template <typename SampleType, typename EdgeArray, typename WeightArray>
  __device__ inline VertexID next(int step, CSRPartition* csr, const VertexID* transit, const VertexID sampleIdx,
                                  SampleType* sample, const float max_weight, EdgeArray& transitEdges,
                                  WeightArray& transitEdgeWeights, const EdgePos_t numEdges,
                                  const VertexID_t neighbrID, curandState* state) {
    EdgePos_t x = RandNumGen::rand_int(state, numEdges);
    sample->previous = *transit;
    sample->stepsTaken++;
    return transitEdges[x];
  }

  __host__ __device__ int samplingType() { return SamplingType::IndividualNeighborhood; }
  __host__ __device__ OutputFormat outputFormat() { return SampledVertices; }
  __host__ __device__ EdgePos_t numSamples(CSR* graph) { return graph->get_n_vertices(); }

  template <class SampleType>
  __host__ std::vector<VertexID_t> initialSample(int sampleIdx, CSR* graph, SampleType& sample) {
    std::vector<VertexID_t> initialValue;
    initialValue.push_back(sampleIdx);
    return initialValue;
  }

  __host__ __device__ EdgePos_t initialSampleSize(CSR* graph) { return 1; }
  __host__ __device__ bool hasExplicitTransits() { return false; }

  template <class SampleType>
  __host__ __device__ VertexID_t stepTransits(int step, const VertexID_t sampleID, SampleType& sample,
                                              int transitIdx, curandState* randState) {
    return -1;
  }

  template <class SampleType>
  __host__ SampleType initializeSample(CSR* graph, const VertexID_t sampleID) {
    SampleType sample;
    sample.previous = -1;
    sample.stepsTaken = 0;
    return sample;
  }
};

// A checker in the style of the reference's app-local ones (src/tests/singleGPU/multirw.cu:11-40,
// src/check_results.cu:46-60): the library's rule on the sampled vertices, then the sample
// states in nextDoorData.samples against the walks in nextDoorData.hFinalSamples.
template <class SampleType, typename App>
bool checkCallerWalkResult(NextDoorData<SampleType, App>& nextDoorData) {
  if (!checkSampledVerticesResult<SampleType, App>(nextDoorData)) return false;
  auto finalSampleSize = getFinalSampleSize<App>();
  auto& finalSamples = nextDoorData.hFinalSamples;
  auto& samples = nextDoorData.samples;
  auto INVALID_VERTEX = nextDoorData.INVALID_VERTEX;
  if (samples.size() * finalSampleSize != finalSamples.size()) {
    printf("%zu sample states for %zu walks\n", samples.size(), finalSamples.size() / finalSampleSize);
    return false;
  }
  for (size_t s = 0; s < samples.size(); s++) {
    int taken = 0;
    while (taken < finalSampleSize && finalSamples[s * finalSampleSize + taken] != INVALID_VERTEX) taken++;
    // the walk stepped once per vertex it holds, the last time from the vertex before its last one
    VertexID_t previous = -1;
    if (taken == 1) previous = nextDoorData.initialContents[s];
    if (taken > 1) previous = finalSamples[s * finalSampleSize + taken - 2];
    if (samples[s].stepsTaken != taken || samples[s].previous != previous) {
      printf("sample %zu: state {%d, %d}, walk says {%d, %d}\n", s, samples[s].previous, samples[s].stepsTaken, previous,
             taken);
      return false;
    }
  }
  printf("sample states checked %zu\n", samples.size());
  return true;
}

// src/tests/testBase.h:14-24, with the gtest scaffolding replaced by a function that returns the result
#define APP_TEST_BINARY(SampleClass, AppName, App, Graph, Path, Runs, CheckResults, chkResultsFunc, KernelType, \
                        LoadBalancing)                                                                           \
  bool AppName##_##Graph(const char* path) {                                                                     \
    bool b = nextdoor<SampleClass, App>(Path, "edge-list", "text", Runs, CheckResults, true, KernelType,         \
                                        LoadBalancing, chkResultsFunc);                                          \
    return b;                                                                                                    \
  }
#define COMMA ,
APP_TEST_BINARY(KHopSample, KHop, KHop3x2App, RingLB, path, 1, true,
                checkSampledVerticesResult<KHopSample COMMA KHop3x2App>, "TransitParallel", true)
APP_TEST_BINARY(KHopSample, KHop, KHop3x2App, RingSP, path, 1, true,
                checkSampledVerticesResult<KHopSample COMMA KHop3x2App>, "SampleParallel", false)

int main(int argc, char* argv[]) {
  if (argc > 2 && strcmp(argv[1], "--registry-app") == 0) return KHop_RingLB(argv[2]) && KHop_RingSP(argv[2]) ? 0 : 1;
  // Call the main function of NextDoor to execute the application (example/uniformRandWalk.cu:95-98)
  return appMain<CallerWalkSample, CallerWalkApp>(argc, argv, checkCallerWalkResult<CallerWalkSample, CallerWalkApp>);
}
