// Fused-activation descriptor; same surface as the reference's
// src/userdriver/common/operator_interfaces/common/ActivationInfo.hpp:3-32.
#pragma once

class ActivationInfo {
public:
    enum class ActivationType { NONE, RELU, RELU1, RELU6, TANH, SIGMOID };

    ActivationInfo() = default;
    ActivationInfo(ActivationType type, const bool &enabled) : type_(type), enabled_(enabled) {}

    ActivationType activation() const { return type_; }
    bool isEnabled() const { return enabled_; }
    bool disable() {
        enabled_ = false;
        return enabled_;
    }

private:
    ActivationType type_ = ActivationType::NONE;
    bool enabled_ = false;
};
