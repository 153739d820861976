// Seeded input generation, preprocessing and number parsing of the `knn` driver.  These define
// the inputs every result is compared on, so they follow the reference exactly:
// generators include/bits/generator/uniform_generator.hpp:42-59 and normal_generator.hpp:42-59
// (std::default_random_engine seeded, 4096 draws discarded, one distribution object per call),
// preprocessors include/bits/preprocessor/ordering_preprocessor.hpp:36-42, number suffixes
// include/bits/utils.hpp:20-74.
#ifndef KNN_HOST_INPUT_HPP_
#define KNN_HOST_INPUT_HPP_

#include <algorithm>
#include <array>
#include <cstddef>
#include <cstdlib>
#include <functional>
#include <random>
#include <stdexcept>
#include <string>
#include <vector>

namespace knn_host
{

// "12", "4k", "1M", "2G": decimal number with an optional binary suffix (2^10, 2^20, 2^30)
inline std::size_t parse_number(std::string text)
{
    if (text.empty())
    {
        return 0;
    }
    std::size_t scale = 1;
    switch (text.back())
    {
    case 'k':
    case 'K':
        scale = std::size_t{1} << 10U;
        break;
    case 'm':
    case 'M':
        scale = std::size_t{1} << 20U;
        break;
    case 'g':
    case 'G':
        scale = std::size_t{1} << 30U;
        break;
    default:
        break;
    }
    if (scale != 1)
    {
        text.pop_back();
    }
    return static_cast<std::size_t>(std::atol(text.c_str())) * scale;
}

// up to three comma separated numbers; missing ones are 1
inline std::array<std::size_t, 3> parse_dim3(const std::string& text)
{
    std::array<std::size_t, 3> values{1, 1, 1};
    std::size_t begin = 0;
    for (std::size_t part = 0;; ++part)
    {
        const std::size_t comma = text.find(',', begin);
        const std::string piece = text.substr(begin, comma == std::string::npos ? comma : comma - begin);
        if (part < 3)
        {
            values[part] = parse_number(piece);
        }
        if (comma == std::string::npos)
        {
            break;
        }
        begin = comma + 1;
    }
    return values;
}

// comma separated floats of a generator specification ("uniform:0,10")
inline std::vector<float> parse_floats(const std::string& text)
{
    std::vector<float> values;
    const char* cursor = text.c_str();
    const char* const end = cursor + text.size();
    while (cursor < end)
    {
        char* next = nullptr;
        const float value = std::strtof(cursor, &next);
        if (next == cursor)
        {
            throw std::invalid_argument("Invalid float parameter");
        }
        if (next + 1 < end && *next != ',')
        {
            throw std::invalid_argument("Invalid parameter format");
        }
        values.push_back(value);
        cursor = next + 1;
    }
    return values;
}

class data_generator
{
public:
    virtual ~data_generator() = default;
    virtual std::string id() const = 0;
    virtual std::vector<float> generate(std::size_t count, std::size_t dim) = 0;
    virtual void set_params(const std::string& params) = 0;

    // seed 0 asks for a non-deterministic seed
    void set_seed(std::size_t seed)
    {
        std::random_device device;
        engine_ = std::default_random_engine{seed == 0 ? device() : seed};
        engine_.discard(1U << 12U);
    }

protected:
    template <typename Distribution>
    std::vector<float> draw(Distribution distribution, std::size_t values)
    {
        std::vector<float> data(values);
        for (float& value : data)
        {
            value = distribution(engine_);
        }
        return data;
    }

    static std::array<float, 2> two_params(const std::string& params, std::array<float, 2> current)
    {
        const auto values = parse_floats(params);
        if (values.size() > 2)
        {
            throw std::invalid_argument("Invalid number of parameters");
        }
        if (values.size() == 2)
        {
            current = {values[0], values[1]};
        }
        else if (values.size() == 1)
        {
            current = {0.0F, values[0]};
        }
        return current;
    }

    std::default_random_engine engine_;
};

class uniform_generator : public data_generator
{
public:
    std::string id() const override { return "uniform"; }
    std::vector<float> generate(std::size_t count, std::size_t dim) override
    {
        return draw(std::uniform_real_distribution<float>{min_, max_}, count * dim);
    }
    void set_params(const std::string& params) override
    {
        const auto range = two_params(params, {min_, max_});
        if (range[0] >= range[1])
        {
            throw std::invalid_argument("Invalid parameter values");
        }
        min_ = range[0];
        max_ = range[1];
    }

private:
    float min_ = 0;
    float max_ = 1;
};

class normal_generator : public data_generator
{
public:
    std::string id() const override { return "normal"; }
    std::vector<float> generate(std::size_t count, std::size_t dim) override
    {
        return draw(std::normal_distribution<float>{mean_, std_dev_}, count * dim);
    }
    void set_params(const std::string& params) override
    {
        const auto values = two_params(params, {mean_, std_dev_});
        if (values[1] <= 0)
        {
            throw std::invalid_argument("Invalid standard deviation");
        }
        mean_ = values[0];
        std_dev_ = values[1];
    }

private:
    float mean_ = 0;
    float std_dev_ = 1;
};

// "identity" leaves the data alone; "ascending" / "descending" zero every query and sort all data
// floats, which makes every row of the distance matrix monotone
inline bool preprocess(const std::string& id, std::vector<float>& data, std::vector<float>& query)
{
    if (id == "identity")
    {
        return true;
    }
    if (id != "ascending" && id != "descending")
    {
        return false;
    }
    std::fill(query.begin(), query.end(), 0.0F);
    if (id == "ascending")
    {
        std::sort(data.begin(), data.end(), std::less<>{});
    }
    else
    {
        std::sort(data.begin(), data.end(), std::greater<>{});
    }
    return true;
}

} // namespace knn_host

#endif // KNN_HOST_INPUT_HPP_
