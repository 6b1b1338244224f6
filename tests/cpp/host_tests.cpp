// Host-only tests (no GPU): expression DSL known answers, cache traces against
// the reference's vectors, and the module stack on the host test device.
#include "check.hpp"
#include "custos/combiner.hpp"
#include "custos/opt_graph.hpp"
#include "module_tests.hpp"
#include "test_cpu_device.hpp"
#include "../../custos_amd/csrc/scratch_order.hpp"

using namespace custos;

// ---- expression DSL: src/two_way_ops/mod.rs:51-202, eval.rs:6-13, resolve.rs:12-23 ----

TEST_CASE(combiner_exp) {
    auto f = [](auto x) { return x.exp(); };
    CHECK_EQ(eval<float>(f(to_val(1.f))), 2.7182817f);  // == core::f32::consts::E
    CHECK_EQ(to_cl_source(f(to_marker<float>("x"))), std::string("exp(x)"));
}
TEST_CASE(combiner_neg_tan) {
    auto f = [](auto x) { return x.tan().neg(); };
    CHECK(std::fabs(eval<float>(f(to_val(2.f))) - 2.1850398f) < 1e-6);
    CHECK_EQ(to_cl_source(f(to_marker<float>("val"))), std::string("-(tan(val))"));
}
TEST_CASE(combiner_pow) {
    auto f = [](auto x, auto y) { return x.mul(3.f).pow(y.add(1.f)); };
    CHECK_EQ(eval<float>(f(to_val(3.f), to_val(2.f))), 729.f);
    CHECK_EQ(to_cl_source(f(to_marker<float>("x"), to_marker<float>("y"))), std::string("pow((x * 3.0), (y + 1.0))"));
}
TEST_CASE(combiner_int_ops) {
    CHECK_EQ(eval<int>(to_val(3).eq(to_val(3))), 1);
    CHECK_EQ(to_cl_source(to_marker<int>("var_x").eq(to_marker<int>("other"))), std::string("(var_x == other)"));
    auto relu = [](auto x) { return x.geq(0).mul(x); };
    CHECK_EQ(eval<int>(relu(to_val(3))), 3);
    CHECK_EQ(to_cl_source(relu(to_marker<int>("var_x"))), std::string("((var_x >= 0) * var_x)"));
    CHECK_EQ(eval<int>(to_val(3).add(3)), 6);
    CHECK_EQ(to_cl_source(to_marker<int>("var_x").add(3)), std::string("(var_x + 3)"));
    CHECK_EQ(eval<int>(to_val(3).geq(4)), 0);
    CHECK_EQ(to_cl_source(to_marker<int>("var_x").geq(4)), std::string("(var_x >= 4)"));
    auto f = [](auto x) { return x.add(2).add(x.mul(8)); };
    CHECK_EQ(eval<int>(f(to_val(4))), 38);
}
TEST_CASE(combiner_two_args_and_strings) {
    auto f = [](auto x, auto y) { return x.add(y).mul(3.6f).sub(y); };
    CHECK(std::fabs(eval<float>(f(to_val(4.f), to_val(3.f))) - 22.2f) < 1e-5);
    CHECK_EQ(to_cl_source(f(to_marker<float>("x"), to_marker<float>("y"))), std::string("(((x + y) * 3.6) - y)"));
    auto g = [](auto x) { return x.add(2.f).mul(x).add(x.mul(8.f)).mul(5.f); };
    CHECK_EQ(to_cl_source(g(Resolve<float>{})), std::string("((((x + 2.0) * x) + (x * 8.0)) * 5.0)"));
    CHECK_EQ(to_cl_source(to_marker<float>("x").add(to_marker<float>("y"))), std::string("(x + y)"));
    CHECK_EQ(eval<float>(to_val(1.5f).add(2.5f).mul(3.5f)), 14.f);
    CHECK_EQ(eval<double>(to_val(1.5).mul(to_val(1.5)).add(2.)), 4.25);
    CHECK_EQ(to_cl_source(to_marker<float>("x").mul(to_marker<float>("x")).add(2.f)), std::string("((x * x) + 2.0)"));
    CHECK_EQ(to_cl_source(to_marker<float>("x").add("1.0")), std::string("(x + 1.0)"));
    CHECK_EQ(to_cl_source(to_marker<float>("x").identity()), std::string("x"));
    CHECK_EQ(to_cl_source(to_marker<float>("x").max(3.f).min(5.f)), std::string("min(max(x, 3.0), 5.0)"));
    CHECK_EQ(to_cl_source(to_marker<float>("x").mul(0.1f).sub(-0.5f)), std::string("((x * 0.1) - -0.5)"));
}
TEST_CASE(combiner_min_max_are_selects) {
    const float nan = std::nanf("");
    CHECK_EQ(eval<float>(to_val(nan).max(1.f)), 1.f);  // NaN > 1 is false -> rhs
    CHECK(std::isnan(eval<float>(to_val(1.f).max(nan))));
    CHECK(!std::signbit(eval<float>(to_val(-0.f).max(0.f))));
    CHECK(std::signbit(eval<float>(to_val(0.f).max(-0.f))));
}
TEST_CASE(fused_source_text) {
    // src/devices/fusing.rs:104-120
    std::vector<std::shared_ptr<UnaryHint<float>>> ops = {
        unary<float>([](auto x) { return x.sin(); }).unary,
        unary<float>([](auto x) { return x.neg(); }).unary,
        unary<float>([](auto x) { return x.cos(); }).unary,
    };
    CHECK_EQ(operations_to_fused_src<float>(ops), std::string("x = sin(x);\nx = -(x);\nx = cos(x);\n"));
}

// ---- cache traces: every vector of src/modules/graph/opt_graph/optimize.rs:137-393,692-805 ----

TEST_CASE(cache_trace_basic) {
    OptGraph g;
    auto a = g.add_leaf(10), b = g.add_leaf(10);
    auto c = g.add_node(10, {a, b});
    auto d = g.add_node(10, {c, c});
    g.add_node(10, {d, b});
    CHECK_VEC_EQ(g.trace_cache_path_raw(g.node(c)), (std::vector<size_t>{3, 4}));
    auto traces = g.cache_traces();
    CHECK_EQ(traces.size(), size_t(1));
    CHECK(traces[0] == (CacheTrace{2, {3, 4}}));
}
TEST_CASE(cache_trace_none_when_two_consumers) {
    OptGraph g;
    auto a = g.add_leaf(10), b = g.add_leaf(10);
    auto c = g.add_node(10, {a, b});
    auto d = g.add_node(10, {c, c});
    g.add_node(10, {d, b});
    g.add_node(10, {c, b});
    CHECK_VEC_EQ(g.trace_cache_path_raw(g.node(c)), (std::vector<size_t>{}));
}
TEST_CASE(cache_trace_2) {
    OptGraph g;
    auto a = g.add_leaf(10), b = g.add_leaf(10), u = g.add_leaf(10);
    auto c = g.add_node(10, {a, b});
    g.add_node(10, {a, u});
    auto d = g.add_node(10, {c, c});
    g.add_node(10, {d, b});
    CHECK_VEC_EQ(g.trace_cache_path_raw(g.node(c)), (std::vector<size_t>{5, 6}));
}
TEST_CASE(cache_trace_break) {
    OptGraph g;
    auto a = g.add_leaf(10), b = g.add_leaf(10);
    auto c = g.add_node(10, {a, b});
    auto d = g.add_node(10, {c, c});
    g.add_node(10, {d, a});
    g.add_node(10, {d, b});
    CHECK(g.is_path_optimizable(g.node(c)));
    CHECK(!g.is_path_optimizable(g.node(d)));
    // the first unoptimizable node still joins the trace, then it ends
    CHECK_VEC_EQ(g.trace_cache_path_raw(g.node(c)), (std::vector<size_t>{3}));
}
// src/modules/graph/opt_graph/optimize.rs:248-275 (test_trace_all)
TEST_CASE(cache_trace_all) {
    OptGraph graph;
    const size_t a = graph.add_leaf(10), b = graph.add_leaf(10);
    const size_t c = graph.add_node(10, {a, b});
    const size_t d = graph.add_node(10, {c, c});
    graph.add_node(10, {d, b});
    auto traces = graph.cache_traces();
    CHECK_EQ(traces.size(), size_t(1));
    CHECK(traces[0] == (CacheTrace{2, {3, 4}}));
}

TEST_CASE(cache_trace_leafed_diff_len) {
    OptGraph g;
    auto a = g.add_leaf(10);
    g.add_node(10, {a, a});
    g.add_leaf(10);
    g.add_leaf(10);
    auto c = g.add_node(10, {a, a});
    auto d = g.add_node(10, {c, c});
    g.add_node(10, {d, a});
    auto traces = g.cache_traces();
    CHECK(traces[0] == (CacheTrace{4, {5, 6}}));
}
TEST_CASE(cache_trace_neural_net) {
    OptGraph g;
    auto inputs = g.add_leaf(100 * 10), targets = g.add_leaf(100);
    auto w1 = g.add_leaf(10 * 64), b1 = g.add_leaf(64), w2 = g.add_leaf(64 * 64), b2 = g.add_leaf(64);
    auto w3 = g.add_leaf(64 * 64), b3 = g.add_leaf(64), w4 = g.add_leaf(64), b4 = g.add_leaf(1);
    auto a1 = g.add_node(100 * 64, {inputs, w1});
    auto a2 = g.add_node(100 * 64, {a1, b1});
    a2 = g.add_node(100 * 64, {a2, a2});
    auto a3 = g.add_node(100 * 64, {a2, w2});
    auto a4 = g.add_node(100 * 64, {a3, b2});
    a4 = g.add_node(100 * 64, {a4, a4});
    auto a5 = g.add_node(100 * 64, {a4, w3});
    auto a6 = g.add_node(100 * 64, {a5, b3});
    a6 = g.add_node(100 * 64, {a6, a6});
    auto a7 = g.add_node(100, {a6, w4});
    auto a8 = g.add_node(100, {a7, b4});
    g.add_node(100, {a8, targets});
    auto traces = g.cache_traces();
    CHECK_EQ(traces.size(), size_t(2));
    CHECK(traces[0] == (CacheTrace{10, {11, 12, 13, 14, 15, 16, 17, 18}}));
    CHECK(traces[1] == (CacheTrace{19, {20, 21}}));
}
TEST_CASE(cache_trace_d) {
    OptGraph g;
    auto a = g.add_leaf(10), b = g.add_leaf(10);
    auto c = g.add_node(10, {a, b});
    auto d = g.add_node(10, {c, c});
    g.add_node(10, {a, d});
    CHECK_VEC_EQ(g.trace_cache_path_raw(g.node(c)), (std::vector<size_t>{3, 4}));
    CHECK(g.is_path_optimizable(g.node(c)) && g.is_path_optimizable(g.node(d)));
    auto traces = g.cache_traces();
    CHECK_EQ(traces.size(), size_t(1));
    CHECK(traces[0] == (CacheTrace{2, {3, 4}}));
}
TEST_CASE(cache_trace_none_in_graph) {
    OptGraph g;
    auto a = g.add_leaf(10), b = g.add_leaf(10);
    auto c = g.add_node(10, {a, b});
    CHECK_VEC_EQ(g.trace_cache_path_raw(g.node(c)), (std::vector<size_t>{}));
    CHECK(g.cache_traces().empty());
}
static OptGraph multiple_traces_graph(bool with_skips) {
    OptGraph g;
    auto a = g.add_leaf(10);
    auto b = g.add_node(10, {a, a});
    g.add_leaf(10);
    auto z = g.add_leaf(10);
    auto c = g.add_node(10, {a, a});
    if (with_skips) g.nodes[c].skip = true;
    auto d = g.add_node(10, {c, c});
    g.add_node(10, {d, a});
    auto f = g.add_node(10, {b, z});
    if (with_skips) g.nodes[f].skip = true;
    g.add_node(10, {f, z});
    return g;
}
TEST_CASE(cache_trace_multiple) {
    auto traces = multiple_traces_graph(false).cache_traces();
    CHECK_EQ(traces.size(), size_t(2));
    CHECK(traces[0] == (CacheTrace{1, {7, 8}}));
    CHECK(traces[1] == (CacheTrace{4, {5, 6}}));
}
TEST_CASE(cache_trace_multiple_with_skips) {
    auto traces = multiple_traces_graph(true).cache_traces();
    CHECK_EQ(traces.size(), size_t(1));
    CHECK(traces[0] == (CacheTrace{5, {6}}));
}

// ---- module stack on the host test device ----

REGISTER_MODULE_TESTS(TestCPU, 1e-12)

TEST_CASE(host_device_frees_everything) {
    size_t live = 0;
    {
        TestCPU<Autograd<Graph<Lazy<Base>>>> dev;
        auto buf = dev.buffer<float>({1.f, 2.f, 3.f}).require_grad();
        auto out = dev.unary_ew(buf, [](auto x) { return x.sin(); }, [](auto x) { return x.cos(); });
        dev.run();
        out.backward();
        live = dev.live_allocations;
        CHECK(live >= 3);
    }
    // the device's destructor ran teardown; buffers freed themselves before
}

// Outputs of operations that run at once are not zero-filled first; lazily retrieved ones are.
TEST_CASE(eager_outputs_skip_the_zero_fill) {
    {
        TestCPU<Base> dev;
        auto buf = dev.buffer<float>({1.f, 2.f, 3.f});
        const size_t before = dev.unzeroed_allocations;
        auto out = dev.apply_fn(buf, [](auto x) { return x.mul(2.f); });
        auto sum = dev.apply_fn2(buf, out, [](auto x, auto y) { return x.add(y); });
        CHECK_EQ(dev.unzeroed_allocations, before + 2);
        CHECK_VEC_EQ(sum.read(), (std::vector<float>{3.f, 6.f, 9.f}));
        auto plain = dev.retrieve<float>(3, buf);       // a plain retrieve stays zeroed
        CHECK_EQ(dev.unzeroed_allocations, before + 2);
        CHECK_VEC_EQ(plain.read(), (std::vector<float>{0.f, 0.f, 0.f}));
    }
    {
        TestCPU<Lazy<Base>> dev;
        auto buf = dev.buffer<float>({1.f, 2.f, 3.f});
        const size_t before = dev.unzeroed_allocations;
        auto out = dev.apply_fn(buf, [](auto x) { return x.mul(2.f); });
        dev.run();
        CHECK_EQ(dev.unzeroed_allocations, before);
        CHECK_VEC_EQ(out.replace().read(), (std::vector<float>{2.f, 4.f, 6.f}));
    }
}

// f32 -> f16 against the definition: the nearest representable value, ties to the even
// significand, found by search over the table of all finite halves (no formula shared with
// the conversion under test).
TEST_CASE(half_conversions_round_to_nearest_even) {
    std::vector<double> table;  // all non-negative finite halves, ascending; index = bit pattern
    for (uint32_t b = 0; b < 0x7c00u; b++) table.push_back(static_cast<double>(detail::f16_bits_to_f32(static_cast<uint16_t>(b))));
    for (size_t i = 1; i < table.size(); i++) CHECK(table[i] > table[i - 1]);
    CHECK_EQ(table[1], std::ldexp(1.0, -24));
    CHECK_EQ(table[0x3c00], 1.0);
    CHECK_EQ(table[0x7bff], 65504.0);
    auto nearest = [&](double v) -> uint16_t {  // v >= 0, finite
        if (v >= 65520.0) return 0x7c00;
        size_t hi = std::lower_bound(table.begin(), table.end(), v) - table.begin();
        if (hi == 0) return 0;
        if (hi == table.size()) return 0x7bff;
        const size_t lo = hi - 1;
        const double dl = v - table[lo], dh = table[hi] - v;
        if (dl < dh) return static_cast<uint16_t>(lo);
        if (dh < dl) return static_cast<uint16_t>(hi);
        return static_cast<uint16_t>((lo & 1) ? hi : lo);
    };
    std::vector<float> cases;
    for (size_t i = 0; i + 1 < table.size(); i++) {  // every midpoint and its f32 neighbours
        const float mid = static_cast<float>((table[i] + table[i + 1]) / 2);
        cases.push_back(mid);
        cases.push_back(std::nextafter(mid, 1e30f));
        cases.push_back(std::nextafter(mid, 0.f));
    }
    uint64_t state = 42;
    for (int i = 0; i < 200000; i++) {  // random bit patterns of finite floats
        state = state * 6364136223846793005ull + 1442695040888963407ull;
        const uint32_t u = static_cast<uint32_t>(state >> 33) % 0x7f800000u;
        cases.push_back(detail::f32_from_bits(u));
    }
    for (float extra : {0.f, 65504.f, 65519.996f, 65520.f, 65536.f, 1e-8f, 2.9802322e-8f, 2.9802326e-8f, 5.9604645e-8f, 3.4e38f})
        cases.push_back(extra);
    size_t wrong = 0;
    for (float c : cases) {
        const uint16_t want = nearest(static_cast<double>(c));
        if (detail::f32_to_f16_bits(c) != want || detail::f32_to_f16_bits(-c) != (want | 0x8000u)) wrong++;
    }
    CHECK_EQ(wrong, size_t(0));
    CHECK_EQ(detail::f32_to_f16_bits(INFINITY), uint16_t(0x7c00));
    CHECK((detail::f32_to_f16_bits(NAN) & 0x7c00) == 0x7c00 && (detail::f32_to_f16_bits(NAN) & 0x3ff) != 0);
    // bf16: ties to even on the 16 dropped bits
    CHECK_EQ(detail::f32_to_bf16_bits(detail::f32_from_bits(0x3F808000u)), uint16_t(0x3F80));
    CHECK_EQ(detail::f32_to_bf16_bits(detail::f32_from_bits(0x3F818000u)), uint16_t(0x3F82));
    CHECK_EQ(detail::f32_to_bf16_bits(detail::f32_from_bits(0x3F808001u)), uint16_t(0x3F81));
    // arithmetic rounds at every operation (src/number.rs:487-676)
    const f16 a(0.1f), b(0.2f);
    CHECK_EQ((a + b).bits, detail::f32_to_f16_bits(float(a) + float(b)));
    CHECK_EQ((a * b).bits, detail::f32_to_f16_bits(float(a) * float(b)));
    CHECK_EQ((-a).bits, uint16_t(a.bits ^ 0x8000));
    CHECK_EQ(eval<f16>(Resolve<f16>::with_val(f16(1.5f)).mul(f16(1.5f)).add(2.f)).bits, f16(4.25f).bits);
    CHECK_EQ(to_cl_source(Resolve<f16>::with_marker("x").mul(f16(0.5f)).exp()), std::string("exp((x * 0.5))"));
}

int main(int argc, char** argv) { return check::run(argc, argv); }

// ---- the shared operand table of the allocation-free merged launch: who waits for whom ----
//
// A model of what the library does with the decisions of ScratchOrder: every handle has a stream
// (a count of the launches issued on it), the GPU's event remembers the stream and position it
// was recorded at, a wait makes a stream depend on that position.  Random creations, calls and
// destructions of up to four handles; before every rewrite of the table, the grid that read the
// table last must be ordered before the rewriting stream's next work: it ran on the same stream,
// or that stream waits for an event recorded on the reader's stream at or behind the reader, or
// the reader's handle was destroyed (which drains its stream first).
TEST_CASE(scratch_table_order_against_a_model_of_streams) {
    using custos_hip::ScratchOrder;
    struct Handle {
        bool alive = false;
        uint64_t issued = 0;       // launches issued on its stream
        uint64_t waits_for[4] = {0, 0, 0, 0};  // per other stream: position this stream has waited for
    };
    uint64_t state = 99;
    auto next = [&](uint64_t below) {
        state = state * 6364136223846793005ull + 1442695040888963407ull;
        return (state >> 33) % below;
    };
    for (int trial = 0; trial < 200; trial++) {
        ScratchOrder order;
        Handle handles[4];
        int event_stream = -1;
        uint64_t event_position = 0;
        int reader = -1;              // handle whose grid read the table last and may still run
        uint64_t reader_position = 0;
        int reuses = 0;
        for (int step = 0; step < 60; step++) {
            const size_t h = next(4);
            Handle& me = handles[h];
            if (!me.alive) {
                me = Handle{};
                me.alive = true;
                if (order.handle_created()) {
                    // recorded on the last user's stream, behind everything it has launched
                    int last = -1;
                    for (int k = 0; k < 4; k++)
                        if (order.last_user == &handles[k]) last = k;
                    CHECK(last >= 0 && handles[last].alive);
                    event_stream = last, event_position = handles[last].issued;
                }
                continue;
            }
            if (next(5) == 0) {
                // destroyed: its stream drains first, so nothing of it is still running
                if (reader == static_cast<int>(h)) reader = -1;
                order.handle_destroyed(&me);
                me.alive = false;
                continue;
            }
            // a call: wait if told to, (maybe) rewrite the table, launch, record if told to
            if (order.must_wait(&me)) {
                CHECK(event_stream >= 0);
                me.waits_for[event_stream] = std::max(me.waits_for[event_stream], event_position);
            }
            if (reader >= 0 && reader != static_cast<int>(h))
                CHECK(me.waits_for[reader] >= reader_position);   // the last reader is ordered before this rewrite
            if (order.still_holds_rows_of(&me)) {
                CHECK(reader == static_cast<int>(h) || reader == -1);  // nobody else used the table in between
                reuses++;
            }
            me.issued++;
            reader = static_cast<int>(h), reader_position = me.issued;
            if (order.launched(&me)) event_stream = static_cast<int>(h), event_position = me.issued;
        }
        int alive = 0;
        for (const Handle& handle : handles) alive += handle.alive;
        CHECK_EQ(order.handles, alive);
        (void)reuses;
    }
}
