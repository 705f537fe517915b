// Overflow-checked arithmetic on non-negative int64 values, used by the window-size calculations.
// A calculation is written as a chain on `Nat`; once any step overflows or sees a negative operand the value is
// poisoned and `ok()` stays false.
#ifndef TILEXR_AMD_CHECKED_MATH_H
#define TILEXR_AMD_CHECKED_MATH_H

#include <cstdint>
#include <limits>

namespace TileXREp {

class Nat {
public:
    Nat() : value_(0), ok_(true) {}
    Nat(int64_t v) : value_(v), ok_(v >= 0) {}   // NOLINT: implicit on purpose

    static Nat Bad() { Nat n; n.ok_ = false; return n; }

    bool ok() const { return ok_; }
    int64_t get() const { return ok_ ? value_ : -1; }

    Nat operator+(Nat rhs) const
    {
        if (!ok_ || !rhs.ok_ || rhs.value_ > std::numeric_limits<int64_t>::max() - value_) {
            return Bad();
        }
        return Nat(value_ + rhs.value_);
    }

    Nat operator*(Nat rhs) const
    {
        if (!ok_ || !rhs.ok_) {
            return Bad();
        }
        if (value_ != 0 && rhs.value_ > std::numeric_limits<int64_t>::max() / value_) {
            return Bad();
        }
        return Nat(value_ * rhs.value_);
    }

    Nat alignUp(int64_t alignment) const
    {
        if (!ok_ || alignment <= 0) {
            return Bad();
        }
        const int64_t rem = value_ % alignment;
        return rem == 0 ? *this : *this + Nat(alignment - rem);
    }

    Nat ceilDiv(int64_t divisor) const
    {
        if (!ok_ || divisor <= 0) {
            return Bad();
        }
        return Nat(value_ / divisor + (value_ % divisor == 0 ? 0 : 1));
    }

private:
    int64_t value_;
    bool ok_;
};

inline Nat Max(Nat a, Nat b)
{
    if (!a.ok() || !b.ok()) {
        return Nat::Bad();
    }
    return a.get() >= b.get() ? a : b;
}

} // namespace TileXREp

#endif // TILEXR_AMD_CHECKED_MATH_H
