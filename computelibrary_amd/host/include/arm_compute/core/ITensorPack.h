// Mirrors arm_compute/core/ITensorPack.h:40-110 of the reference: the (slot id -> tensor) map a stateless operator runs on.
#ifndef ACL_MI355_CORE_ITENSORPACK_H
#define ACL_MI355_CORE_ITENSORPACK_H

#include "arm_compute/core/ITensor.h"
#include "arm_compute/core/experimental/Types.h"

#include <initializer_list>
#include <unordered_map>

namespace arm_compute
{
class ITensorPack
{
public:
    struct PackElement
    {
        PackElement() = default;
        PackElement(int id, ITensor *tensor) : id(id), tensor(tensor), ctensor(nullptr) {}
        PackElement(int id, const ITensor *ctensor) : id(id), tensor(nullptr), ctensor(ctensor) {}
        int            id{-1};
        ITensor       *tensor{nullptr};
        const ITensor *ctensor{nullptr};
    };

    ITensorPack() = default;
    ITensorPack(std::initializer_list<PackElement> l)
    {
        for (auto &e : l)
            _pack[e.id] = e;
    }
    void add_tensor(int id, ITensor *tensor) { _pack[id] = PackElement(id, tensor); }
    void add_tensor(int id, const ITensor *tensor) { _pack[id] = PackElement(id, tensor); }
    void add_const_tensor(int id, const ITensor *tensor) { add_tensor(id, tensor); }
    ITensor *get_tensor(int id)
    {
        auto it = _pack.find(id);
        return it != _pack.end() ? it->second.tensor : nullptr;
    }
    const ITensor *get_const_tensor(int id) const
    {
        auto it = _pack.find(id);
        if (it == _pack.end())
            return nullptr;
        return it->second.ctensor != nullptr ? it->second.ctensor : it->second.tensor;
    }
    void   remove_tensor(int id) { _pack.erase(id); }
    size_t size() const { return _pack.size(); }
    bool   empty() const { return _pack.empty(); }

private:
    std::unordered_map<int, PackElement> _pack{};
};
} // namespace arm_compute
#endif
