// Minimal host core: exception hierarchy with the names and roles of include/armnn/Exceptions.hpp:46-158.
#pragma once
#include <sstream>
#include <stdexcept>
#include <string>

namespace armnn
{
struct CheckLocation
{
    const char* m_Function;
    const char* m_File;
    unsigned int m_Line;
    CheckLocation(const char* func, const char* file, unsigned int line) : m_Function{func}, m_File{file}, m_Line{line} {}
    std::string AsString() const
    {
        std::stringstream ss;
        ss << " at function " << m_Function << " [" << m_File << ':' << m_Line << "]";
        return ss.str();
    }
    std::string FileLine() const
    {
        std::stringstream ss;
        ss << " [" << m_File << ':' << m_Line << "]";
        return ss.str();
    }
};
#define CHECK_LOCATION() armnn::CheckLocation(__func__, __FILE__, __LINE__)

class Exception : public std::exception
{
public:
    explicit Exception(const std::string& message) : m_Message{message} {}
    explicit Exception(const std::string& message, const CheckLocation& location) : m_Message{message + location.AsString()} {}
    const char* what() const noexcept override { return m_Message.c_str(); }
private:
    std::string m_Message;
};

#define ARMNN_CORE_EXCEPTION(NAME, BASE)                                                           \
    class NAME : public BASE { public: using BASE::BASE; }
ARMNN_CORE_EXCEPTION(InvalidArgumentException, Exception);
ARMNN_CORE_EXCEPTION(RuntimeException, Exception);
ARMNN_CORE_EXCEPTION(BackendUnavailableException, Exception);
ARMNN_CORE_EXCEPTION(NullPointerException, Exception);
ARMNN_CORE_EXCEPTION(MemoryValidationException, Exception);
ARMNN_CORE_EXCEPTION(MemoryImportException, Exception);
ARMNN_CORE_EXCEPTION(UnimplementedException, Exception);
ARMNN_CORE_EXCEPTION(LayerValidationException, InvalidArgumentException);
ARMNN_CORE_EXCEPTION(GraphValidationException, Exception);
ARMNN_CORE_EXCEPTION(BadOptionalAccessException, Exception);
ARMNN_CORE_EXCEPTION(FileNotFoundException, Exception);
ARMNN_CORE_EXCEPTION(ParseException, Exception);
#undef ARMNN_CORE_EXCEPTION
} // namespace armnn
