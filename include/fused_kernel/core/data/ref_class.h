#ifndef FK_AMD_REF_CLASS_H
#define FK_AMD_REF_CLASS_H
#include <stdexcept>
namespace fk {
// Copy-counted base for handle owners (streams).  Like the reference's (FK/core/data/ref_class.h) the count is
// a plain int: copying one object from two threads at once is not supported.
class Ref {
    struct Count { int n{0}; };
    Count* count_{nullptr};
    void share(const Ref& other) {
        if (other.count_) { count_ = other.count_; ++count_->n; }
    }
    void drop() {
        if (count_ && --count_->n == 0) delete count_;
        count_ = nullptr;
    }
public:
    Ref() : count_(new Count) { count_->n = 1; }
    Ref(const Ref& other) { share(other); }
    Ref(Ref&&) = delete;
    Ref& operator=(Ref&&) = delete;
    Ref& operator=(const Ref& other) {
        if (this != &other) { drop(); share(other); }
        return *this;
    }
    virtual ~Ref() { drop(); }
    // Number of live copies INCLUDING this one while it is alive.
    int getRefCount() const { return count_ ? count_->n : 0; }
};
} // namespace fk
#endif
