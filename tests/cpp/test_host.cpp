// Host-side test of pink::Trainer<..., true> / pink::Mapper<..., true> over the C ABI.
// Mirrors the reference's own tests (paths relative to the reference tree):
//   test/SelfOrganizingMapTest/Trainer.cpp:22-151, Mapper.cpp:80-100, circular_ed.cpp:23-53,
//   test/CudaTest/mapper.cu:55-120.
// Usage: test_host args   -> argument validation only (no device needed)
//        test_host gpu    -> everything
#define PINK_HIP_STANDALONE
#include "pink_hip_som.h"

#include <cmath>
#include <cstdio>
#include <cstring>
#include <numeric>

using namespace pink;

static int failures = 0;
#define EXPECT(cond) do { if (!(cond)) { std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); ++failures; } } while (0)

template <typename F>
static bool throws_pink(F&& f)
{
    try { f(); } catch (pink::exception const&) { return true; } catch (...) { return false; }
    return false;
}

typedef SOM<CartesianLayout<2>, CartesianLayout<2>, float> SOM2;
typedef Trainer<CartesianLayout<2>, CartesianLayout<2>, float, true> Trainer2;
typedef Mapper<CartesianLayout<2>, CartesianLayout<2>, float, true> Mapper2;
typedef Data<CartesianLayout<2>, float> Data2;

static void test_arguments()
{
    SOM2 som({{2, 2}}, {{2, 2}}, 0.0f);
    auto f = GaussianFunctor(1.1f, 0.2f);
    for (uint32_t bad : {0u, 3u, 90u})
        EXPECT(throws_pink([&] { Trainer2(som, f, 0, bad, false, 1.0, Interpolation::BILINEAR, 2); }));
    EXPECT(throws_pink([&] { Mapper2(som, 0, 3, false, Interpolation::BILINEAR, 2); }));
    EXPECT(throws_pink([&] { Mapper2(som, 0, 4, false, Interpolation::BILINEAR, 3); }));   // region larger than neuron
    EXPECT(!throws_pink([&] { Trainer2(som, f, 0, 720, false, 1.0, Interpolation::BILINEAR, 2); }));
    EXPECT(throws_pink([] { HexagonalLayout(HexagonalLayout::DimensionType{{4, 4}}); }));
    EXPECT(HexagonalLayout(HexagonalLayout::DimensionType{{21, 21}}).size() == 331);
}

static void test_trainer()
{
    {   // Trainer.cpp:49-69 (float instead of int weights: 290.1...)
        SOM2 som({{2, 2}}, {{2, 2}}, std::vector<float>(16, 0.0f));
        Trainer2 trainer(som, GaussianFunctor(1.1f, 0.2f), 0, 1, false, 0.0, Interpolation::BILINEAR, 2);
        trainer(Data2({{2, 2}}, {1000, 2000, 3000, 4000}));
        trainer.update_som();
        EXPECT(static_cast<int>(som.get_data_pointer()[3]) == 290);
        EXPECT(trainer.get_update_info()[0] == 1);
    }
    {   // Trainer.cpp:71-94
        SOM2 som({{1, 1}}, {{2, 2}}, std::vector<float>(4, 0.0f));
        Trainer2 trainer(som, StepFunctor(10.0f), 0, 1, false, 0.0, Interpolation::BILINEAR, 2);
        std::vector<float> img(16);
        std::iota(img.begin(), img.end(), 1.0f);
        trainer(Data2({{4, 4}}, img));
        trainer.update_som();
        float const expect[4] = {6, 7, 10, 11};
        EXPECT(std::memcmp(som.get_data_pointer(), expect, sizeof expect) == 0);
    }
    {   // Trainer.cpp:96-124 (3-dimensional data)
        typedef SOM<CartesianLayout<2>, CartesianLayout<3>, float> SOM3;
        std::vector<float> raw(32, 0.0f), rot1{4, 3, 2, 1, 8, 7, 6, 5}, img(8);
        std::copy(rot1.begin(), rot1.end(), raw.begin() + 8);
        std::iota(img.begin(), img.end(), 1.0f);
        SOM3 som({{2, 2}}, {{2, 2, 2}}, raw);
        Trainer<CartesianLayout<2>, CartesianLayout<3>, float, true> trainer(som, StepFunctor(0.0f), 0, 4, false, 0.0,
            Interpolation::BILINEAR, 2);
        trainer(Data<CartesianLayout<3>, float>({{2, 2, 2}}, img));
        trainer.update_som();
        EXPECT(std::memcmp(som.get_data_pointer() + 8, rot1.data(), 8 * sizeof(float)) == 0);
        EXPECT(trainer.get_update_info()[1] == 1);
    }
    {   // hexagonal SOM, two images of different size through one trainer
        typedef SOM<HexagonalLayout, CartesianLayout<2>, float> SOMH;
        SOMH som(HexagonalLayout(HexagonalLayout::DimensionType{{3, 3}}), {{4, 4}}, 0.5f);
        Trainer<HexagonalLayout, CartesianLayout<2>, float, true> trainer(som, GaussianFunctor(1.1f, 0.2f), 0, 8, true,
            -1.0, Interpolation::BILINEAR, 4, EuclideanDistanceShape::QUADRATIC, 256, DataType::UINT8);
        trainer(Data2({{6, 6}}, std::vector<float>(36, 1.0f)));
        trainer(Data2({{8, 8}}, std::vector<float>(64, 1.0f)));
        trainer.update_som();
        EXPECT(som.get_data_pointer()[5] > 0.5f and som.get_data_pointer()[5] < 1.0f);
        auto info = trainer.get_update_info();
        uint32_t total = 0;
        for (uint32_t i = 0; i < 7; ++i) total += info[i];
        EXPECT(total == 2);
    }
}

static void test_mapper()
{
    struct Case { uint32_t som_dim, neuron_dim, image_dim, ed; uint32_t num_rot; bool flip; };
    for (Case c : {Case{1, 2, 2, 2, 1, false}, Case{1, 3, 3, 2, 1, false}, Case{1, 3, 3, 2, 360, false},
                   Case{2, 3, 3, 2, 360, false}, Case{2, 3, 3, 2, 360, true}}) {
        for (DataType t : {DataType::FLOAT, DataType::UINT8, DataType::UINT16}) {   // mapper.cu:115-119
            SOM2 som({{c.som_dim, c.som_dim}}, {{c.neuron_dim, c.neuron_dim}}, 1.0f);
            Mapper2 mapper(som, 0, c.num_rot, c.flip, Interpolation::BILINEAR, c.ed, EuclideanDistanceShape::QUADRATIC, 256, t);
            auto result = mapper(Data2({{c.image_dim, c.image_dim}}, 0.0f));
            for (float v : std::get<0>(result)) EXPECT(v == 2.0f);
        }
    }
    {   // circular_ed.cpp:23-53
        std::vector<float> image(16, 0.0f), som_vec(64, 0.0f);
        image[4] = 1.0f;
        som_vec[4] = 1.0f; som_vec[18] = 0.5f; som_vec[43] = 0.8f; som_vec[61] = 0.3f;
        SOM2 som({{2, 2}}, {{4, 4}}, som_vec);
        Mapper2 mapper(som, 0, 4, false, Interpolation::BILINEAR, 4, EuclideanDistanceShape::CIRCULAR);
        auto result = mapper(Data2({{4, 4}}, image));
        float const expect[4] = {0.0f, 0.5f, 0.2f, 0.7f};
        for (int i = 0; i < 4; ++i) {
            EXPECT(std::fabs(std::get<0>(result)[i] - expect[i]) < 0.01f);
            EXPECT(std::get<1>(result)[i] == static_cast<uint32_t>(i));
        }
    }
}

int main(int argc, char** argv)
{
    bool const gpu = argc > 1 and std::strcmp(argv[1], "gpu") == 0;
    test_arguments();
    if (gpu) {
        test_trainer();
        test_mapper();
    }
    std::printf("%s (%d failures)\n", failures ? "FAILED" : "OK", failures);
    return failures ? 1 : 0;
}
