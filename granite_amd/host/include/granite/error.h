// Error reporting of the Granite API: ErrorCode, Error, Result<T> and the
// propagation macros (reference: include/granite/error.h:16-257).  No
// exceptions cross the API; every fallible call returns a Result.
#pragma once

#include <optional>
#include <source_location>
#include <string>
#include <utility>
#include <variant>

namespace granite {

// Same order as the reference so numeric values agree.
enum class ErrorCode {
    Success = 0,
    FileNotFound, InvalidFormat, IOError,
    OutOfMemory, AllocationFailed, BufferTooSmall,
    BackendNotSupported, BackendNotInitialized, OperatorNotImplemented, ShaderCompilationFailed,
    ExecutionFailed, Timeout,
    InvalidShape, ShapeMismatch, DTypeMismatch, InvalidArgument, NullPointer,
    InvalidGraph, CycleDetected, InvalidState,
    UnsupportedModel, CorruptedWeights, MissingOperator,
    InternalError, NotImplemented,
};

constexpr const char* error_code_name(ErrorCode c) {
    constexpr const char* names[] = {
        "Success", "FileNotFound", "InvalidFormat", "IOError", "OutOfMemory", "AllocationFailed",
        "BufferTooSmall", "BackendNotSupported", "BackendNotInitialized", "OperatorNotImplemented",
        "ShaderCompilationFailed", "ExecutionFailed", "Timeout", "InvalidShape", "ShapeMismatch",
        "DTypeMismatch", "InvalidArgument", "NullPointer", "InvalidGraph", "CycleDetected",
        "InvalidState", "UnsupportedModel", "CorruptedWeights", "MissingOperator", "InternalError",
        "NotImplemented"};
    const auto i = static_cast<size_t>(c);
    return i < sizeof(names) / sizeof(names[0]) ? names[i] : "Unknown";
}

class Error {
  public:
    Error(ErrorCode code, std::string message,
          std::source_location where = std::source_location::current())
        : code_(code), message_(std::move(message)), where_(where) {}
    Error(ErrorCode code, std::source_location where = std::source_location::current())
        : code_(code), message_(error_code_name(code)), where_(where) {}

    [[nodiscard]] ErrorCode code() const { return code_; }
    [[nodiscard]] const std::string& message() const { return message_; }
    [[nodiscard]] const std::source_location& location() const { return where_; }
    [[nodiscard]] std::string to_string() const {
        return std::string(error_code_name(code_)) + ": " + message_ + " (at " +
               where_.file_name() + ":" + std::to_string(where_.line()) + ")";
    }

  private:
    ErrorCode code_;
    std::string message_;
    std::source_location where_;
};

template <typename T>
class Result {
  public:
    Result(T value) : data_(std::move(value)) {}
    Result(Error error) : data_(std::move(error)) {}
    Result(ErrorCode code, std::source_location where = std::source_location::current())
        : data_(Error(code, where)) {}

    [[nodiscard]] bool ok() const { return std::holds_alternative<T>(data_); }
    explicit operator bool() const { return ok(); }
    [[nodiscard]] T& value() & { return std::get<T>(data_); }
    [[nodiscard]] const T& value() const& { return std::get<T>(data_); }
    [[nodiscard]] T&& value() && { return std::get<T>(std::move(data_)); }
    [[nodiscard]] T take() { return std::get<T>(std::move(data_)); }
    [[nodiscard]] const Error& error() const { return std::get<Error>(data_); }
    [[nodiscard]] T value_or(T fallback) const { return ok() ? std::get<T>(data_) : fallback; }

    template <typename F>
    auto map(F&& f) -> Result<decltype(f(std::declval<T>()))> {
        using U = decltype(f(std::declval<T>()));
        if (ok()) return Result<U>(f(std::get<T>(data_)));
        return Result<U>(std::get<Error>(data_));
    }
    template <typename F>
    auto and_then(F&& f) -> decltype(f(std::declval<T>())) {
        if (ok()) return f(std::get<T>(data_));
        return decltype(f(std::declval<T>()))(std::get<Error>(data_));
    }

  private:
    std::variant<T, Error> data_;
};

template <>
class Result<void> {
  public:
    Result() = default;
    Result(Error error) : error_(std::move(error)) {}
    Result(ErrorCode code, std::source_location where = std::source_location::current())
        : error_(Error(code, where)) {}
    [[nodiscard]] bool ok() const { return !error_.has_value(); }
    explicit operator bool() const { return ok(); }
    [[nodiscard]] const Error& error() const { return error_.value(); }

  private:
    std::optional<Error> error_;
};

#define GRANITE_TRY(expr)                                      \
    do {                                                       \
        auto _granite_result = (expr);                         \
        if (!_granite_result.ok()) return _granite_result.error(); \
    } while (0)

#define GRANITE_TRY_ASSIGN(var, expr)                                        \
    auto _granite_result_##var = (expr);                                     \
    if (!_granite_result_##var.ok()) return _granite_result_##var.error();   \
    auto var = std::move(_granite_result_##var).take()

#define GRANITE_ERROR(code, msg) ::granite::Error((code), (msg), std::source_location::current())
#define GRANITE_FAIL(code, msg) return GRANITE_ERROR(code, msg)

}  // namespace granite
