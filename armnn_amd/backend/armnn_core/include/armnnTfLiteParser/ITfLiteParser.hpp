// TfLite front end of the host core: a quantized .tflite model becomes an INetwork
// (include/armnnTfLiteParser/ITfLiteParser.hpp:1-96 is the interface this mirrors).
#pragma once
#include <armnn/INetwork.hpp>
#include <armnn/Optional.hpp>
#include <armnn/Tensor.hpp>

#include <memory>
#include <string>
#include <vector>

namespace armnnTfLiteParser
{
using BindingPointInfo = armnn::BindingPointInfo;

class TfLiteParserImpl;
class ITfLiteParser;
using ITfLiteParserPtr = std::unique_ptr<ITfLiteParser, void (*)(ITfLiteParser* parser)>;

class ITfLiteParser
{
public:
    struct TfLiteParserOptions
    {
        bool m_AllowExpandedDims = false;
        bool m_StandInLayerForUnsupported = false;      // not offered: an operator outside the list is a ParseException
        bool m_InferAndValidate = false;
    };

    static ITfLiteParser* CreateRaw(const armnn::Optional<TfLiteParserOptions>& options = armnn::EmptyOptional());
    static ITfLiteParserPtr Create(const armnn::Optional<TfLiteParserOptions>& options = armnn::EmptyOptional());
    static void Destroy(ITfLiteParser* parser);

    /// Create the network from a flatbuffers binary file on disk
    armnn::INetworkPtr CreateNetworkFromBinaryFile(const char* graphFile);
    /// Create the network from a flatbuffers binary
    armnn::INetworkPtr CreateNetworkFromBinary(const std::vector<uint8_t>& binaryContent);

    /// Binding id and tensor info of the network input / output with this tensor name
    BindingPointInfo GetNetworkInputBindingInfo(size_t subgraphId, const std::string& name) const;
    BindingPointInfo GetNetworkOutputBindingInfo(size_t subgraphId, const std::string& name) const;

    size_t GetSubgraphCount() const;
    std::vector<std::string> GetSubgraphInputTensorNames(size_t subgraphId) const;
    std::vector<std::string> GetSubgraphOutputTensorNames(size_t subgraphId) const;

private:
    explicit ITfLiteParser(const armnn::Optional<TfLiteParserOptions>& options);
    ~ITfLiteParser();
    std::unique_ptr<TfLiteParserImpl> pTfLiteParserImpl;
};
} // namespace armnnTfLiteParser
