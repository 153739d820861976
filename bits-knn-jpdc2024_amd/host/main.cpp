// `knn`: the benchmark driver.  Same command line, phases, CSV rows on stdout and `Checksum:`
// lines on stderr as the reference driver (src/main.cpp:83-102 log format, :168-207 options,
// :291-343 input generation, :366-437 phase loop); the algorithms it registers are the ones of
// the k-NN hot path (algorithms.cpp).
#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdint>
#include <exception>
#include <functional>
#include <iomanip>
#include <iostream>
#include <limits>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "input.hpp"
#include "knn.hpp"

namespace
{

struct option_spec
{
    char short_name; // 0 when there is none
    const char* long_name;
    const char* description;
    const char* default_value; // nullptr for flags
};

const std::vector<option_spec>& option_table()
{
    static const std::vector<option_spec> table{
        {'a', "algorithm", "Used algorithm", "serial"},
        {'r', "repeat", "Number of executions", "1"},
        {'k', "knn", "Number of nearest neighbors", "1"},
        {'n', "number", "Number of objects in the database", "1024"},
        {'q', "query", "Number of query objects", "1024"},
        {'d', "dimension", "Dimension of objects", "1"},
        {'g', "generator", "Data generator", "uniform"},
        {'p', "preprocessor", "Data preprocessor", "identity"},
        {0, "seed", "Seed for the data generator", "0"},
        {0, "block-size", "Block size for GPU kernels", "256"},
        {0, "items-per-thread",
         "Further arguments for the algorithm; up to three comma-separated numbers", "1"},
        {'v', "verify", "Verify the results against selected implementation", "off"},
        {0, "point-layout",
         "Layout of the point matrix - \"column\" for column major or \"row\" for row major", "row"},
        {0, "query-layout",
         "Layout of the query matrix - \"column\" for column major or \"row\" for row major", "row"},
        {0, "deg", "degree of parallelism used for single-query problems", "1"},
        {0, "no-output", "Do not copy the result back to CPU", nullptr},
        {0, "header", "Print header with column names and exit", nullptr},
        {'h', "help", "Show help message and exit", nullptr},
    };
    return table;
}

class command_line
{
public:
    command_line(int argc, char** argv)
    {
        for (int i = 1; i < argc; ++i)
        {
            const std::string arg = argv[i];
            const option_spec* spec = nullptr;
            std::string inline_value;
            bool has_inline = false;
            if (arg.rfind("--", 0) == 0)
            {
                const auto eq = arg.find('=');
                const std::string name = arg.substr(2, eq == std::string::npos ? eq : eq - 2);
                spec = find([&](const option_spec& o) { return name == o.long_name; });
                if (eq != std::string::npos)
                {
                    inline_value = arg.substr(eq + 1);
                    has_inline = true;
                }
            }
            else if (arg.size() >= 2 && arg[0] == '-')
            {
                spec = find([&](const option_spec& o) { return o.short_name != 0 && arg[1] == o.short_name; });
                if (arg.size() > 2)
                {
                    inline_value = arg.substr(2);
                    has_inline = true;
                }
            }
            if (spec == nullptr)
            {
                throw std::invalid_argument("Option '" + arg + "' does not exist");
            }
            if (spec->default_value == nullptr)
            {
                values_[spec->long_name] = "true";
            }
            else if (has_inline)
            {
                values_[spec->long_name] = inline_value;
            }
            else
            {
                if (i + 1 >= argc)
                {
                    throw std::invalid_argument("Option '" + arg + "' is missing an argument");
                }
                values_[spec->long_name] = argv[++i];
            }
        }
    }

    bool given(const std::string& name) const { return values_.count(name) != 0; }

    std::string get(const std::string& name) const
    {
        const auto it = values_.find(name);
        if (it != values_.end())
        {
            return it->second;
        }
        const option_spec* spec = find([&](const option_spec& o) { return name == o.long_name; });
        return spec != nullptr && spec->default_value != nullptr ? spec->default_value : "";
    }

private:
    template <typename Pred>
    static const option_spec* find(Pred pred)
    {
        for (const auto& option : option_table())
        {
            if (pred(option))
            {
                return &option;
            }
        }
        return nullptr;
    }

    std::map<std::string, std::string> values_;
};

void print_help(const std::vector<std::unique_ptr<knn>>& algorithms)
{
    std::cerr << "kNN\nUsage:\n  knn [OPTION...]\n\n";
    for (const auto& option : option_table())
    {
        std::string left = "  ";
        left += option.short_name != 0 ? std::string{"-"} + option.short_name + ", " : std::string{"    "};
        left += std::string{"--"} + option.long_name + (option.default_value != nullptr ? " arg" : "");
        left.resize(std::max<std::size_t>(left.size() + 2, 30), ' ');
        std::cerr << left << option.description;
        if (option.default_value != nullptr)
        {
            std::cerr << " (default: " << option.default_value << ")";
        }
        std::cerr << '\n';
    }
    std::cerr << '\n' << "Available algorithms:" << '\n';
    for (const auto& algorithm : algorithms)
    {
        std::cerr << "- " << algorithm->id() << "\n";
    }
}

void print_header()
{
    std::cout << "algorithm,generator,preprocessor,iteration,point_count,query_count,dim,"
                 "block_size,k,items_per_thread,deg,phase,time"
              << '\n';
}

struct run_labels
{
    std::string algorithm;
    std::string generator;
    std::string preprocessor;
};

// one CSV row per phase and iteration
void log_phase(const knn_args& args, const run_labels& labels, const char* phase,
               std::size_t iteration, double seconds)
{
    const auto precision = std::cout.precision();
    std::cout << labels.algorithm << ',' << labels.generator << ',' << labels.preprocessor << ','
              << iteration << ',' << args.point_count << ',' << args.query_count << ',' << args.dim
              << ',' << args.selection_block_size << ',' << args.k << ",\"" << args.items_per_thread[0]
              << ',' << args.items_per_thread[1] << ',' << args.items_per_thread[2] << "\","
              << args.deg << ',' << phase << ',' << std::scientific
              << std::setprecision(std::numeric_limits<double>::digits10 + 1) << seconds
              << std::defaultfloat << std::setprecision(static_cast<int>(precision)) << '\n';
}

template <typename Phase>
double timed(Phase&& phase)
{
    const auto begin = std::chrono::steady_clock::now();
    phase();
    const std::chrono::duration<double> elapsed = std::chrono::steady_clock::now() - begin;
    return elapsed.count();
}

std::vector<float> transposed(const std::vector<float>& matrix, std::size_t rows, std::size_t cols)
{
    std::vector<float> out(matrix.size());
    for (std::size_t i = 0; i < rows; ++i)
    {
        for (std::size_t j = 0; j < cols; ++j)
        {
            out[j * rows + i] = matrix[i * cols + j];
        }
    }
    return out;
}

knn* find_algorithm(const std::vector<std::unique_ptr<knn>>& algorithms, const std::string& id)
{
    for (const auto& algorithm : algorithms)
    {
        if (algorithm->id() == id)
        {
            return algorithm.get();
        }
    }
    return nullptr;
}

int run(int argc, char** argv)
{
    const auto algorithms = make_algorithms();
    const command_line cli{argc, argv};

    if (cli.given("help"))
    {
        print_help(algorithms);
        return 0;
    }
    if (cli.given("header"))
    {
        print_header();
        return 0;
    }

    using knn_host::parse_number;
    const std::size_t dim = parse_number(cli.get("dimension"));
    const std::size_t k = parse_number(cli.get("knn"));
    const std::size_t point_count = parse_number(cli.get("number"));
    const std::size_t query_count = parse_number(cli.get("query"));
    const std::size_t repeat = parse_number(cli.get("repeat"));
    const std::size_t seed = parse_number(cli.get("seed"));
    const std::size_t block_size = parse_number(cli.get("block-size"));
    const std::string verify_id = cli.get("verify");
    run_labels labels{cli.get("algorithm"), cli.get("generator"), cli.get("preprocessor")};

    if (dim == 0)
    {
        std::cerr << "Dimension must be greater than 0" << '\n';
        return 1;
    }
    if (point_count == 0)
    {
        std::cerr << "Number of objects in the database must be greater than 0" << '\n';
        return 1;
    }
    if (query_count == 0)
    {
        std::cerr << "Number of query objects must be greater than 0" << '\n';
        return 1;
    }
    if (k == 0)
    {
        std::cerr << "Number of nearest neighbors must be greater than 0" << '\n';
        return 1;
    }
    if (block_size == 0)
    {
        std::cerr << "Block size must be greater than 0" << '\n';
        return 1;
    }

    // "uniform:0,10" -> generator id and its parameters
    std::string generator_params;
    const auto colon = labels.generator.find(':');
    const bool has_params = colon != std::string::npos;
    if (has_params)
    {
        generator_params = labels.generator.substr(colon + 1);
        labels.generator = labels.generator.substr(0, colon);
    }
    knn_host::uniform_generator uniform;
    knn_host::normal_generator normal;
    knn_host::data_generator* generator = nullptr;
    for (knn_host::data_generator* candidate : {static_cast<knn_host::data_generator*>(&uniform),
                                                static_cast<knn_host::data_generator*>(&normal)})
    {
        if (candidate->id() == labels.generator)
        {
            generator = candidate;
        }
    }
    if (generator == nullptr)
    {
        std::cerr << "Unknown generator: '" << labels.generator << "'" << '\n';
        return 1;
    }
    generator->set_seed(seed);
    if (has_params)
    {
        generator->set_params(generator_params);
    }

    // points first, then queries, from the same engine
    std::vector<float> data = generator->generate(point_count, dim);
    std::vector<float> query = generator->generate(query_count, dim);
    if (!knn_host::preprocess(labels.preprocessor, data, query))
    {
        std::cerr << "Unknown preprocessor: '" << labels.preprocessor << "'" << '\n';
        return 1;
    }

    knn_args args;
    args.point_count = point_count;
    args.query_count = query_count;
    args.dim = dim;
    args.points_layout = cli.get("point-layout") == "row" ? matrix_layout::row_major : matrix_layout::column_major;
    args.queries_layout = cli.get("query-layout") == "row" ? matrix_layout::row_major : matrix_layout::column_major;
    args.dist_layout = matrix_layout::row_major;
    args.dist_block_size = block_size;
    args.selection_block_size = block_size;
    args.k = k;
    args.items_per_thread = knn_host::parse_dim3(cli.get("items-per-thread"));
    args.deg = parse_number(cli.get("deg"));
    if (args.points_layout == matrix_layout::column_major)
    {
        data = transposed(data, point_count, dim);
    }
    if (args.queries_layout == matrix_layout::column_major)
    {
        query = transposed(query, query_count, dim);
    }
    args.points = data.data();
    args.queries = query.data();

    knn* const algorithm = find_algorithm(algorithms, labels.algorithm);
    if (algorithm == nullptr)
    {
        std::cerr << "Unknown algorithm: '" << labels.algorithm << "'" << '\n';
        print_help(algorithms);
        return 1;
    }
    const bool no_output = cli.given("no-output");
    if (no_output)
    {
        algorithm->no_output();
    }
    algorithm->initialize(args);

    for (std::size_t iteration = 0; iteration < repeat; ++iteration)
    {
        log_phase(args, labels, "prepare", iteration, timed([&] { algorithm->prepare(); }));
        log_phase(args, labels, "transfer-in", iteration, algorithm->transfer_in_seconds());
        log_phase(args, labels, "distances", iteration, timed([&] { algorithm->distances(); }));
        log_phase(args, labels, "selection", iteration, timed([&] { algorithm->selection(); }));
        log_phase(args, labels, "postprocessing", iteration, timed([&] { algorithm->postprocessing(); }));
        std::vector<distance_pair> result;
        log_phase(args, labels, "finish", iteration, timed([&] { result = algorithm->finish(); }));
        log_phase(args, labels, "transfer-out", iteration, algorithm->transfer_out_seconds());

        if (!no_output)
        {
            // sum of the neighbour indices of query 0, modulo 2^32
            std::uint32_t checksum = 0;
            for (std::size_t j = 0; j < k && j < result.size(); ++j)
            {
                checksum += static_cast<std::uint32_t>(result[j].index);
            }
            std::cerr << "Checksum: " << checksum << '\n';
        }

        if (cli.given("verify"))
        {
            knn* const other = find_algorithm(algorithms, verify_id);
            if (other != nullptr)
            {
                other->initialize(args);
                other->prepare();
                other->distances();
                other->selection();
                verify(other->finish(), result, k);
            }
        }
    }
    return 0;
}

} // namespace

int main(int argc, char** argv)
{
    try
    {
        return run(argc, argv);
    }
    catch (const std::exception& error)
    {
        std::cerr << error.what() << '\n';
        return 1;
    }
    catch (...)
    {
        std::cerr << "Unknown exception" << '\n';
        return 1;
    }
}
