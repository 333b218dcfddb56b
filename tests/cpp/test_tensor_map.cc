// Host-side semantics of Tensor / TensorMap, as the reference defines them
// (src/fastertransformer/utils/Tensor.h:286-504, utils/Tensor.cc:334-377). No GPU involved.
#include <cstdio>
#include <stdexcept>
#include <string>

#include "src/fastertransformer/utils/Tensor.h"

using namespace fastertransformer;

static int failures = 0;
#define EXPECT(cond)                                                                                                   \
    do {                                                                                                               \
        if (!(cond)) {                                                                                                 \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);                                              \
            ++failures;                                                                                                \
        }                                                                                                              \
    } while (0)

template<typename F>
static bool throws_runtime_error(F f)
{
    try {
        f();
    }
    catch (const std::runtime_error&) {
        return true;
    }
    catch (...) {
        return false;
    }
    return false;
}

int main()
{
    float  data[12] = {0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11};
    int    one      = 7;
    Tensor t(MEMORY_CPU, TYPE_FP32, {3, 4}, data);
    Tensor null_data(MEMORY_CPU, TYPE_FP32, {3, 4}, nullptr);
    Tensor empty(MEMORY_CPU, TYPE_FP32, {}, data);

    EXPECT(t.size() == 12);
    EXPECT(t.sizeBytes() == 48);
    EXPECT(t.getVal<float>(5) == 5.0f);
    EXPECT(t.getPtr<float>() == data);
    EXPECT(getTensorType<float>() == TYPE_FP32 && getTensorType<half>() == TYPE_FP16
           && getTensorType<bfloat16>() == TYPE_BF16 && getTensorType<const int*>() != TYPE_INT32);

    // list / map constructors silently drop tensors without data or without elements
    TensorMap m({{"a", t}, {"null", null_data}, {"empty", empty}});
    EXPECT(m.size() == 1 && m.isExist("a") && !m.isExist("null") && !m.isExist("empty"));
    // insert(key, tensor) refuses them, and refuses duplicates
    EXPECT(throws_runtime_error([&] { m.insert("null", null_data); }));
    EXPECT(throws_runtime_error([&] { m.insert("a", t); }));
    // insert(pair) does not check: an output key may exist with a null pointer
    m.insert({"null", null_data});
    EXPECT(m.isExist("null") && m.at("null").data == nullptr);
    m.insertIfValid("empty", empty);
    EXPECT(!m.isExist("empty"));
    // lookups
    EXPECT(throws_runtime_error([&] { m.at("missing"); }));
    EXPECT(m.at("missing", t).data == data);
    EXPECT(m.getVal<int>("missing", 3) == 3);
    m.insert("one", Tensor(MEMORY_CPU, TYPE_INT32, {1}, &one));
    EXPECT(m.getVal<int>("one") == 7 && m.getVal<int>("one", 3) == 7);

    // slice: bounds-checked pointer offset, passes a null pointer through
    Tensor s = t.slice({2, 4}, 4);
    EXPECT(s.getPtr<float>() == data + 4 && s.size() == 8);
    EXPECT(throws_runtime_error([&] { t.slice({3, 4}, 4); }));
    EXPECT(null_data.slice({1, 4}, 4).data == nullptr);

    std::printf(failures == 0 ? "OK\n" : "%d failure(s)\n", failures);
    return failures == 0 ? 0 : 1;
}
