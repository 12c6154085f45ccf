// Compile check of the Llaminar-side binding (include/llaminar_amd/binding/) against the
// reference's own interface headers, where the reference tree is present.  Never linked and
// never run: tests/test_binding_compiles.py passes this file to the compiler with
// -fsyntax-only.  Each adapter is instantiated through a pointer to the interface it
// implements, so a pure virtual left unimplemented (ITensorGemm, IWorkspaceConsumer,
// IMoEKernel, IPackedWeights) or a signature that no longer overrides anything fails here.
#include <llaminar_amd/binding/MI355MoEAdapter.h>
#include <llaminar_amd/binding/MI355QuantGemmAdapter.h>

#include <memory>
#include <type_traits>

using namespace llaminar2;

static_assert(!std::is_abstract<mi355::MI355QuantGemmAdapter>::value, "MI355QuantGemmAdapter leaves a pure virtual open");
static_assert(!std::is_abstract<mi355::MI355MoEAdapter>::value, "MI355MoEAdapter leaves a pure virtual open");
static_assert(!std::is_abstract<mi355::MI355PackedWeightsHandle>::value, "MI355PackedWeightsHandle leaves a pure virtual open");
static_assert(std::is_base_of<ITensorGemm, mi355::MI355QuantGemmAdapter>::value, "not an ITensorGemm");
static_assert(std::is_base_of<IWorkspaceConsumer, mi355::MI355QuantGemmAdapter>::value, "not an IWorkspaceConsumer");
static_assert(std::is_base_of<IMoEKernel, mi355::MI355MoEAdapter>::value, "not an IMoEKernel");

// what the load pipeline does with a weight tensor (loaders/PreparedWeightStore.h:68-79)
std::shared_ptr<ITensorGemm> make_gemm(const TensorBase *w, int rocm_ordinal)
{
    return std::make_shared<mi355::MI355QuantGemmAdapter>(w, rocm_ordinal);
}
std::unique_ptr<IWorkspaceConsumer> make_consumer(const void *host_rows)
{
    return std::make_unique<mi355::MI355QuantGemmAdapter>(LLAM_FMT_Q4_K, host_rows, 256, 256, 0);
}
std::unique_ptr<IMoEKernel> make_moe(int rocm_ordinal) { return std::make_unique<mi355::MI355MoEAdapter>(rocm_ordinal); }

// the calls the stages make, through the interfaces, with the interfaces' default arguments
bool calls(ITensorGemm *g, IMoEKernel *m, DeviceWorkspaceManager *ws, const TensorBase *a, TensorBase *c,
           DeviceMoELayerRuntime *rt, ITensor *ids, ITensor *wts)
{
    std::vector<ITensorGemm::TensorProjectionDesc> projs{{g, c, g->get_n()}};
    ITensorGemm::FusedExpertDownDesc down{g, nullptr, nullptr, g->get_n()};
    DeviceNativeVNNIMatrixDesc desc;
    auto *consumer = dynamic_cast<IWorkspaceConsumer *>(g);
    consumer->bindWorkspace(ws);
    g->prepareWeights();
    bool ok = g->multiply_tensor(a, c, 1, g->get_n(), g->get_k()) && g->multiply_tensor(a, c) &&
              g->multiply_tensor_with_fused_swiglu(a, a, c, 1, g->get_n(), g->get_k()) &&
              g->multiply_fused_tensor(a, projs, 1, g->get_k()) &&
              g->multiply_fused_verifier_rows_decode_equivalent(a, projs, 2, g->get_k()) &&
              g->multiply_fused_expert_down(&down, 1, 1, g->get_k()) && g->exportNativeVNNIMatrixDesc(desc) &&
              g->multiply_with_precomputed_q8_1(nullptr, nullptr, 1, g->get_n(), g->get_k()) &&
              consumer->hasWorkspace() && consumer->getWorkspace() == ws &&
              consumer->getWorkspaceRequirements(8).total_bytes() > 0;
    std::unique_ptr<IPackedWeights> w = g->detachWeights();
    ok = ok && g->attachWeights(std::move(w));
    const int t = m->uploadGroupedExpertGateUpDescriptorTables(&desc, &desc, 1, g->get_k(), g->get_n());
    const int d = m->uploadGroupedExpertDownDescriptorTable(&desc, 1, g->get_k(), g->get_n());
    ok = ok && m->decodeRouteSelect(rt, c, c, g->get_k(), 256, 8, true, ids, wts, true, true) &&
         m->groupedExpertDecodeFromRuntime(rt, a, t, d, 8, c, g->get_k(), g->get_n());
    return ok;
}
