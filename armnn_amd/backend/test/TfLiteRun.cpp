// A .tflite model through ITfLiteParser -> INetwork -> Optimize -> IRuntime::LoadNetwork -> IRuntime::EnqueueWorkload.
// Usage:
//   tflite_run <model.tflite> <input bytes file, or - for seeded bytes> <output bytes file> <backends, e.g. Mi355x or Mi355x,CpuRef> [iterations]
// Prints one JSON line: the parsed bindings, the optimized graph layer by layer (type, name, backend) and the time per
// inference.  Builds against this repository's host core and, unchanged, against an Arm NN source tree and its
// libarmnn.so (then together with RealGraphAccess.cpp and the parser source, which uses the public INetwork API only).
#include <armnn/ArmNN.hpp>
#include <armnnTfLiteParser/ITfLiteParser.hpp>
#include <Graph.hpp>
#include <Layer.hpp>

#include <chrono>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <iterator>
#include <sstream>

using namespace armnn;

int main(int argc, char** argv)
{
    if (argc < 5)
    {
        std::fprintf(stderr, "usage: %s <model.tflite> <input bytes | -> <output bytes> <backends> [iterations]\n", argv[0]);
        return 2;
    }
    const int iterations = argc > 5 ? std::atoi(argv[5]) : 1;
    try
    {
        ConfigureLogging(true, false, LogSeverity::Error);
        armnnTfLiteParser::ITfLiteParserPtr parser = armnnTfLiteParser::ITfLiteParser::Create();
        INetworkPtr net = parser->CreateNetworkFromBinaryFile(argv[1]);
        const std::vector<std::string> inNames = parser->GetSubgraphInputTensorNames(0), outNames = parser->GetSubgraphOutputTensorNames(0);
        if (inNames.size() != 1 || outNames.size() != 1) throw std::runtime_error("one input and one output are expected");
        const armnnTfLiteParser::BindingPointInfo in = parser->GetNetworkInputBindingInfo(0, inNames[0]);
        const armnnTfLiteParser::BindingPointInfo out = parser->GetNetworkOutputBindingInfo(0, outNames[0]);

        std::vector<uint8_t> input(in.second.GetNumBytes());
        if (std::strcmp(argv[2], "-") == 0)
        {
            uint64_t s = 88172645463325252ull;
            for (auto& v : input) { s ^= s << 13; s ^= s >> 7; s ^= s << 17; v = static_cast<uint8_t>(s); }
        }
        else
        {
            std::ifstream f(argv[2], std::ios::binary);
            std::vector<uint8_t> bytes((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
            if (bytes.size() != input.size()) throw std::runtime_error("input file size does not match the model's input");
            input = bytes;
        }

        std::vector<BackendId> backends;
        std::stringstream list(argv[4]);
        for (std::string b; std::getline(list, b, ',');) backends.emplace_back(b);
        IRuntimePtr rt = IRuntime::Create(IRuntime::CreationOptions());
        IOptimizedNetworkPtr opt = Optimize(*net, backends, rt->GetDeviceSpec());
        std::string layers;
        for (auto&& l : GetGraphForTesting(opt.get()))
        {
            if (!layers.empty()) layers += ", ";
            layers += std::string("[\"") + GetLayerTypeAsCString(l->GetType()) + "\", \"" + l->GetNameStr() + "\", \"" + l->GetBackendId().Get() + "\"]";
        }
        NetworkId id = 0;
        std::string err;
        if (rt->LoadNetwork(id, std::move(opt), err) != Status::Success) throw std::runtime_error("LoadNetwork: " + err);
        TensorInfo cin = in.second;
        cin.SetConstant(true);
        std::vector<uint8_t> output(out.second.GetNumBytes());
        const InputTensors ins{{in.first, ConstTensor(cin, input.data())}};
        const OutputTensors outs{{out.first, Tensor(out.second, output.data())}};
        if (rt->EnqueueWorkload(id, ins, outs) != Status::Success) throw std::runtime_error("EnqueueWorkload failed");
        const auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < iterations; ++i)
            if (rt->EnqueueWorkload(id, ins, outs) != Status::Success) throw std::runtime_error("EnqueueWorkload failed");
        const double ms = 1e3 * std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() / std::max(1, iterations);
        std::ofstream fo(argv[3], std::ios::binary);
        fo.write(reinterpret_cast<const char*>(output.data()), static_cast<std::streamsize>(output.size()));
        auto shape = [](const TensorInfo& t) {
            std::string s = "[";
            for (unsigned int i = 0; i < t.GetNumDimensions(); ++i) s += (i ? ", " : "") + std::to_string(t.GetShape()[i]);
            return s + "]";
        };
        std::printf("{\"input\": \"%s\", \"input_binding\": %d, \"input_shape\": %s, \"output\": \"%s\", \"output_binding\": %d, \"output_shape\": %s, "
                    "\"ms_per_inference\": %.4f, \"layers\": [%s]}\n",
                    inNames[0].c_str(), static_cast<int>(in.first), shape(in.second).c_str(), outNames[0].c_str(), static_cast<int>(out.first),
                    shape(out.second).c_str(), ms, layers.c_str());
        rt->UnloadNetwork(id);
        return 0;
    }
    catch (const std::exception& e)
    {
        std::fprintf(stderr, "tflite_run: %s\n", e.what());
        return 1;
    }
}
