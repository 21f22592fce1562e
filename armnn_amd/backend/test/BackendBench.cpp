// Throughput of a network through the backend, the way an Arm NN application runs it:
//   INetwork -> Optimize({"Mi355x"}) -> IRuntime::LoadNetwork -> IRuntime::EnqueueWorkload, host buffers in and out.
// Usage:
//   backend_bench <network file> <input bytes file> <output bytes file> [steps] [warmup] [backends, default Mi355x]
// The network file comes from armnn_amd/netfile.py.  Prints one JSON line: milliseconds per EnqueueWorkload with
// pageable host buffers (two host copies and the staging transfers) and with adopted pinned buffers (ImportInputs /
// ImportOutputs, one transfer each way), the layer counts of the optimized graph, and whether both runs gave the same
// bytes.  The output of the last run is written to the output file for the caller to compare.  With a backend list that
// does not name Mi355x (CpuRef on the reference's runtime: the CPU baseline) only the pageable figure is measured.
// Builds against this repository's host core and, unchanged, against an Arm NN source tree and its libarmnn.so (then
// together with RealGraphAccess.cpp, which supplies the test utilities' GetGraphForTesting).
#include <armnn/ArmNN.hpp>
#include <Graph.hpp>
#include <Layer.hpp>

#include <armnn_mi355x.h>

#include <chrono>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <iterator>
#include <sstream>

#include "NetFile.hpp"
#include "../mi355x/Mi355xWorkloads.hpp"

using namespace armnn;

namespace
{
size_t Count(const Graph& g, LayerType t)
{
    size_t n = 0;
    for (auto&& l : g) n += l->GetType() == t;
    return n;
}
} // namespace

int main(int argc, char** argv)
{
    if (argc < 4)
    {
        std::fprintf(stderr, "usage: %s <network file> <input bytes> <output bytes> [steps] [warmup]\n", argv[0]);
        return 2;
    }
    const int steps = argc > 4 ? std::atoi(argv[4]) : 200;
    const int warmup = argc > 5 ? std::atoi(argv[5]) : 10;
    const std::string backendList = argc > 6 ? argv[6] : "Mi355x";
    try
    {
        const netfile::Net nf = netfile::Read(argv[1]);
        std::ifstream fin(argv[2], std::ios::binary);
        std::vector<uint8_t> input((std::istreambuf_iterator<char>(fin)), std::istreambuf_iterator<char>());
        const TensorInfo inInfo = nf.tensors.at(nf.input);
        const TensorInfo outInfo = nf.tensors.at(nf.output);
        if (input.size() != inInfo.GetNumBytes()) throw std::runtime_error("input file size does not match the network's input");

        ConfigureLogging(true, false, LogSeverity::Error);
        IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
        INetworkPtr net = netfile::Build(nf);
        std::vector<BackendId> backends;
        std::stringstream list(backendList);
        for (std::string b; std::getline(list, b, ',');) backends.emplace_back(b);
        const bool onDevice = backendList.find("Mi355x") != std::string::npos;
        IOptimizedNetworkPtr opt = Optimize(*net, backends, rt->GetDeviceSpec());
        const Graph& og = GetGraphForTesting(opt.get());
        const size_t nLayers = og.GetNumLayers(), nAct = Count(og, LayerType::Activation), nCopy = Count(og, LayerType::MemCopy),
                     nConv = Count(og, LayerType::Convolution2d), nDw = Count(og, LayerType::DepthwiseConvolution2d),
                     nAdd = Count(og, LayerType::ElementwiseBinary);
        NetworkId id = -1;
        std::string err;
        if (rt->LoadNetwork(id, std::move(opt), err) != Status::Success) throw std::runtime_error("LoadNetwork: " + err);

        TensorInfo constIn = inInfo;
        constIn.SetConstant(true);
        std::vector<uint8_t> pageable(outInfo.GetNumBytes());
        InputTensors ins{{0, ConstTensor(constIn, input.data())}};
        OutputTensors outs{{0, Tensor(outInfo, pageable.data())}};
        for (int i = 0; i < warmup; ++i)
            if (rt->EnqueueWorkload(id, ins, outs) != Status::Success) throw std::runtime_error("EnqueueWorkload failed");
        auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < steps; ++i)
            if (rt->EnqueueWorkload(id, ins, outs) != Status::Success) throw std::runtime_error("EnqueueWorkload failed");
        const double msPageable = 1e3 * std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() / steps;

        if (!onDevice)
        {
            std::ofstream fout(argv[3], std::ios::binary);
            fout.write(reinterpret_cast<const char*>(pageable.data()), static_cast<std::streamsize>(pageable.size()));
            rt->UnloadNetwork(id);
            std::printf("{\"batch\": %u, \"steps\": %d, \"backends\": \"%s\", \"ms_pageable\": %.4f, \"optimized_layers\": %zu}\n", nf.batch, steps,
                        backendList.c_str(), msPageable, nLayers);
            return 0;
        }
        void *pin = nullptr, *pout = nullptr;
        if (mi355x_host_alloc(&pin, input.size()) != 0 || mi355x_host_alloc(&pout, pageable.size()) != 0) throw std::runtime_error(mi355x_last_error());
        std::memcpy(pin, input.data(), input.size());
        const auto inIds = rt->ImportInputs(id, {{0, ConstTensor(constIn, pin)}}, MemorySource::Malloc);
        const auto outIds = rt->ImportOutputs(id, {{0, Tensor(outInfo, pout)}}, MemorySource::Malloc);
        if (inIds.size() != 1 || outIds.size() != 1)
            throw std::runtime_error("pinned buffers were not adopted: " + std::to_string(inIds.size()) + " of 1 inputs, " + std::to_string(outIds.size()) + " of 1 outputs");
        for (int i = 0; i < warmup; ++i)
            if (rt->EnqueueWorkload(id, {}, {}, inIds, outIds) != Status::Success) throw std::runtime_error("EnqueueWorkload failed");
        t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < steps; ++i)
            if (rt->EnqueueWorkload(id, {}, {}, inIds, outIds) != Status::Success) throw std::runtime_error("EnqueueWorkload failed");
        const double msPinned = 1e3 * std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() / steps;
        const bool same = std::memcmp(pout, pageable.data(), pageable.size()) == 0;

        // input and output resident on the device (adopted device memory): what one inference costs without the bus
        double msDevice = 0.0;
        bool deviceSame = true;
        void *din = nullptr, *dout = nullptr;
        {
            if (mi355x_malloc(&din, input.size()) != 0 || mi355x_malloc(&dout, pageable.size()) != 0) throw std::runtime_error(mi355x_last_error());
            if (mi355x_memcpy_h2d(din, input.data(), input.size(), nullptr) != 0 || mi355x_device_synchronize() != 0) throw std::runtime_error(mi355x_last_error());
            const auto dinIds = rt->ImportInputs(id, {{0, ConstTensor(constIn, din)}}, MemorySource::Malloc);
            const auto doutIds = rt->ImportOutputs(id, {{0, Tensor(outInfo, dout)}}, MemorySource::Malloc);
            if (dinIds.size() == 1 && doutIds.size() == 1)
            {
                for (int i = 0; i < warmup; ++i)
                    if (rt->EnqueueWorkload(id, {}, {}, dinIds, doutIds) != Status::Success) throw std::runtime_error("EnqueueWorkload failed");
                mi355x_device_synchronize();
                t0 = std::chrono::steady_clock::now();
                for (int i = 0; i < steps; ++i)
                    if (rt->EnqueueWorkload(id, {}, {}, dinIds, doutIds) != Status::Success) throw std::runtime_error("EnqueueWorkload failed");
                mi355x_device_synchronize();
                msDevice = 1e3 * std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() / steps;
                std::vector<uint8_t> back(pageable.size());
                if (mi355x_memcpy_d2h(back.data(), dout, back.size(), nullptr) != 0 || mi355x_device_synchronize() != 0) throw std::runtime_error(mi355x_last_error());
                deviceSame = back == pageable;
            }
            mi355x_device_synchronize();
        }

        std::ofstream fout(argv[3], std::ios::binary);
        fout.write(static_cast<const char*>(pout), static_cast<std::streamsize>(pageable.size()));
        rt->UnloadNetwork(id);
        mi355x_host_free(pin);
        mi355x_host_free(pout);
        mi355x_free(din);
        mi355x_free(dout);
        std::printf("{\"batch\": %u, \"steps\": %d, \"ms_pageable\": %.4f, \"ms_pinned\": %.4f, \"ms_device_resident\": %.4f, \"pinned_equals_pageable\": %s, "
                    "\"optimized_layers\": %zu, \"activation_layers_left\": %zu, \"memcopy_layers\": %zu, \"conv_layers\": %zu, "
                    "\"depthwise_layers\": %zu, \"add_layers\": %zu, \"additions_running_a_convolution\": %llu}\n",
                    nf.batch, steps, msPageable, msPinned, msDevice, (same && deviceSame) ? "true" : "false", nLayers, nAct, nCopy, nConv, nDw, nAdd, Mi355xAdditionWorkload::PairsFormed());
        return (same && deviceSame) ? 0 : 1;
    }
    catch (const std::exception& e)
    {
        std::fprintf(stderr, "backend_bench: %s\n", e.what());
        return 1;
    }
}
