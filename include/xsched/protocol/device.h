// XDevice packing: device type in the high word, 32-bit PCI id in the low word
// (reference protocol/src/device.cpp:6-19; PCI id layout utils/include/xsched/utils/pci.h).
#pragma once

#include "xsched/types.h"

namespace xsched::protocol
{

inline XDeviceId   GetDeviceId(XDevice dev)   { return (XDeviceId)(dev & 0xFFFFFFFFull); }
inline XDeviceType GetDeviceType(XDevice dev) { return (XDeviceType)(dev >> 32); }
inline XDevice MakeDevice(XDeviceType type, XDeviceId id)
{
    return ((uint64_t)type << 32) | (uint64_t)id;
}

// domain:16 | bus:8 | device:5 | function:3
inline XDeviceId MakePciId(uint32_t domain, uint32_t bus, uint32_t device, uint32_t function)
{
    return ((domain & 0xFFFF) << 16) | ((bus & 0xFF) << 8) | ((device & 0x1F) << 3) | (function & 0x7);
}

} // namespace xsched::protocol
