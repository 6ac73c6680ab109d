// C++ harness over es_km.hpp in the style of the reference's kernel-manager experiments
// (exps/gpuexec_kernelmanager.cc:18-160, exps/cpuexec_kernels.cc:9-86): build an einsummable,
// fill inputs from a seeded std::mt19937 the way dbuffer_t::random does
// (src/einsummable/dbuffer.cc:198-229), run it through kernel_manager_t on device buffers,
// and compare with the CPU oracle.  Exits non-zero on the first mismatch.
#include "es_km.hpp"
#include "es_oracle.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cmath>
#include <condition_variable>
#include <mutex>
#include <cstdio>
#include <random>

using namespace eskm;

#define HIP_OK(x)                                                                      \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            std::printf("FAIL hip: %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
            std::exit(2);                                                              \
        }                                                                              \
    } while (0)

struct device_buffer_t {
    void*  ptr = nullptr;
    size_t bytes;
    explicit device_buffer_t(size_t n) : bytes(n) { HIP_OK(hipMalloc(&ptr, n ? n : 1)); }
    ~device_buffer_t() { (void)hipFree(ptr); }
    void upload(void const* src) { HIP_OK(hipMemcpy(ptr, src, bytes, hipMemcpyHostToDevice)); }
    void download(void* dst) { HIP_OK(hipMemcpy(dst, ptr, bytes, hipMemcpyDeviceToHost)); }
};

static std::vector<float> random_f32(std::mt19937& gen, size_t n, float lo, float hi)
{
    std::uniform_real_distribution<float> dist(lo, hi);
    std::vector<float>                    v(n);
    for (auto& x : v) x = dist(gen);
    return v;
}

static std::vector<uint16_t> random_f16(std::mt19937& gen, size_t n, float lo, float hi)
{
    std::uniform_real_distribution<float> dist(lo, hi);
    std::vector<uint16_t>                 v(n);
    for (auto& x : v) x = es_oracle_f32_to_f16(dist(gen));
    return v;
}

static void expect(bool ok, const char* what)
{
    if (!ok) {
        std::printf("FAIL %s\n", what);
        std::exit(1);
    }
    std::printf("ok   %s\n", what);
}

static std::vector<int> flatten(einsummable_t const& e, std::vector<int>& offs)
{
    std::vector<int> flat;
    offs.assign(1, 0);
    for (auto const& inn : e.inns) {
        flat.insert(flat.end(), inn.begin(), inn.end());
        offs.push_back(int(flat.size()));
    }
    return flat;
}

static void oracle_run(einsummable_t const& e, void* out, std::vector<void const*> inns)
{
    std::vector<int> offs;
    std::vector<int> flat = flatten(e, offs);
    int rc = es_oracle_einsummable(e.join_shape.data(), int(e.join_shape.size()), flat.data(),
                                   offs.data(), int(e.inns.size()), e.out_rank, e.join.c_str(),
                                   castable_char(e.castable), ES_O_WIDE, out, inns.data());
    if (rc) {
        std::printf("FAIL oracle: %s\n", es_oracle_last_error());
        std::exit(1);
    }
}

int main()
{
    HIP_OK(hipSetDevice(0));
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    std::mt19937     gen(0);
    kernel_manager_t km(0);

    {  // test_mm: f32 matmul through from_matmul (exps/cpuexec_kernels.cc:9-33)
        uint64_t      ni = 200, nj = 136, nk = 72;
        einsummable_t e = einsummable_t::from_matmul(ni, nj, nk, dtype_t::f32);
        auto          lhs = random_f32(gen, ni * nj, -1, 1), rhs = random_f32(gen, nj * nk, -1, 1);
        std::vector<float> ref(ni * nk), got(ni * nk);
        oracle_run(e, ref.data(), {lhs.data(), rhs.data()});
        auto ws = km.build(e);
        expect(ws.has_value() && km.workspace_size(e).value() == ws.value().value(), "build matmul");
        device_buffer_t dl(lhs.size() * 4), dr(rhs.size() * 4), dout(got.size() * 4),
            dws(ws.value().value());
        dl.upload(lhs.data());
        dr.upload(rhs.data());
        km(e, stream, dout.ptr, {dl.ptr, dr.ptr}, std::make_tuple(dws.ptr, ws.value().value()));
        HIP_OK(hipStreamSynchronize(stream));
        dout.download(got.data());
        double worst = 0;
        for (size_t i = 0; i != got.size(); ++i) worst = std::max(worst, std::fabs(double(got[i]) - ref[i]));
        expect(worst <= 1e-4 * 8.0, "matmul f32 200x136x72 within 1e-4 of its magnitude");
    }

    {  // silu on f16 (exps/gpuexec_kernelmanager.cc, llama/modules.cc:416)
        uint64_t      n = 10000;
        einsummable_t e{{n}, {{0}}, 1,
                        "*[hole|f16@0,power{-1}[+[constant{f16|1},exp[*[constant{f16|-1},hole|f16@0]]]]]",
                        std::nullopt};
        auto          x = random_f16(gen, n, -4, 4);
        std::vector<uint16_t> ref(n), got(n);
        oracle_run(e, ref.data(), {x.data()});
        expect(km.build(e).has_value(), "build silu");
        device_buffer_t dx(n * 2), dout(n * 2);
        dx.upload(x.data());
        km(e, stream, dout.ptr, {dx.ptr});
        HIP_OK(hipStreamSynchronize(stream));
        dout.download(got.data());
        double worst = 0;
        for (size_t i = 0; i != n; ++i) {
            double a = es_oracle_f16_to_f32(got[i]), b = es_oracle_f16_to_f32(ref[i]);
            worst = std::max(worst, std::fabs(a - b) / std::max(std::fabs(b), 1.0));
        }
        expect(worst <= 1e-2, "silu f16 within 1e-2");
    }

    {  // touch with castable add: exact (exps/cpuexec_touch.cc:85-114)
        touch_t t{{{16, 64, 0, 8, 16}, {16, 64, 0, 24, 16}}, castable_t::add, dtype_t::f32};
        auto    inn = random_f32(gen, 256, -1, 1), out = random_f32(gen, 4096, -1, 1);
        std::vector<float> ref = out, got(4096);
        es_oracle_touch(reinterpret_cast<uint64_t const*>(t.selection.data()), 2, '+', ES_O_F32,
                        ref.data(), inn.data());
        device_buffer_t di(256 * 4), dout(4096 * 4);
        di.upload(inn.data());
        dout.upload(out.data());
        km(t, stream, dout.ptr, di.ptr);
        HIP_OK(hipStreamSynchronize(stream));
        dout.download(got.data());
        expect(std::memcmp(got.data(), ref.data(), 4096 * 4) == 0, "touch add bit exact");
    }

    {  // fills
        fill_t::lowertri_t l{scalar_t(0.0f), scalar_t(-INFINITY), 40, 56, 3};
        std::vector<float> ref(40 * 56), got(40 * 56);
        es_oracle_fill_lowertri(ES_O_F32, l.lower.bits(), l.upper.bits(), 40, 56, 3, ref.data());
        device_buffer_t d(ref.size() * 4);
        km.lowerTri_fill(l, stream, d.ptr);
        HIP_OK(hipStreamSynchronize(stream));
        d.download(got.data());
        expect(std::memcmp(got.data(), ref.data(), ref.size() * 4) == 0, "lowerTri_fill bit exact");
        fill_t::constant_t c{scalar_t(2.5), {7, 11}};
        std::vector<double> gc(77);
        device_buffer_t     dc(77 * 8);
        km.constant_fill(c, stream, dc.ptr);
        HIP_OK(hipStreamSynchronize(stream));
        dc.download(gc.data());
        bool all = true;
        for (double v : gc) all = all && v == 2.5;
        expect(all, "constant_fill");
    }

    {  // error behaviour (gpu_kernel_manager.cc:957, 1103-1107, 1260)
        einsummable_t unbuilt{{33}, {{0}}, 1, "exp[hole|f32@0]", std::nullopt};
        device_buffer_t d(33 * 4);
        bool threw = false;
        try {
            km(unbuilt, stream, d.ptr, {d.ptr});
        } catch (std::runtime_error const&) {
            threw = true;
        }
        expect(threw, "executing an un-built einsummable throws");
        einsummable_t with_var{{33}, {{0}}, 1, "*[variable{lr|f32},hole|f32@0]", std::nullopt};
        expect(!km.build(with_var).has_value(), "unsupported einsummable builds to nullopt");
        km.build(unbuilt);
        threw = false;
        try {
            km(unbuilt, stream, d.ptr, {d.ptr, d.ptr});
        } catch (std::runtime_error const&) {
            threw = true;
        }
        expect(threw, "wrong input count throws");
    }

    {  // exec-node layer: out = relu(x) + relu(y) as three dependent nodes over one arena,
       // a grouped pair of touches, on two streams (src/engine/gpu/exec_graph.cc:258-404)
        uint64_t const n = 4096, B = n * 4;
        std::string const relu = "ite_>=[constant{f32|0},hole|f32@0,constant{f32|0},hole|f32@0]";
        einsummable_t e_relu{{n}, {{0}}, 1, relu, std::nullopt};
        einsummable_t e_add{{n}, {{0}, {0}}, 1, "+[hole|f32@0,hole|f32@1]", std::nullopt};
        auto x = random_f32(gen, n, -1, 1), y = random_f32(gen, n, -1, 1);
        device_buffer_t arena(6 * B);
        std::vector<float> host(6 * n, 9.0f), got(6 * n);
        std::copy(x.begin(), x.end(), host.begin());
        std::copy(y.begin(), y.end(), host.begin() + n);
        arena.upload(host.data());
        exec_graph_t g(km);
        int a = g.insert_einsummable(e_relu, {{2 * B, B}, {0, B}});
        int b = g.insert_einsummable(e_relu, {{3 * B, B}, {B, B}});
        int c = g.insert_einsummable(e_add, {{4 * B, B}, {2 * B, B}, {3 * B, B}}, {a, b});
        touch_t t{{{n, n, 0, 0, n}}, castable_t::add, dtype_t::f32};
        g.insert_touch(t, 0, {5 * B, B}, {0, B});          // first of its group: initialises
        g.insert_touch(t, 0, {5 * B, B}, {4 * B, B}, {c});  // accumulates
        g.finalize(2);
        g.run(stream, arena.ptr);
        HIP_OK(hipStreamSynchronize(stream));
        arena.download(got.data());
        bool ok = true;
        for (uint64_t i = 0; i != n; ++i) {
            float s = std::max(x[i], 0.0f) + std::max(y[i], 0.0f);
            ok = ok && got[4 * n + i] == s && got[5 * n + i] == x[i] + s;
        }
        expect(ok, "exec graph: dependent nodes and a touch group on two streams");
    }

    {  // host storage (gpu_evict_t / gpu_load_t) and a serialized memgraph
       // (memgraph_t::from_wire): inputmem, alloc, relu as an apply node, evict, load
        uint64_t const n = 1024, B = n * 4;
        auto x = random_f32(gen, n, -1, 1);
        device_buffer_t arena(3 * B);
        std::vector<float> host(3 * n, 5.0f), got(3 * n), slot(n);
        std::copy(x.begin(), x.end(), host.begin());
        arena.upload(host.data());
        auto varint = [](uint64_t v) {
            std::string o;
            do {
                o.push_back(char((v & 0x7f) | (v > 0x7f ? 0x80 : 0)));
                v >>= 7;
            } while (v);
            return o;
        };
        auto scalar = [&](int f, uint64_t v) { return varint(uint64_t(f) << 3) + varint(v); };
        auto bytes = [&](int f, std::string const& b) {
            return varint(uint64_t(f) << 3 | 2) + varint(b.size()) + b;
        };
        auto los = [&](uint64_t off) { return scalar(1, 0) + scalar(2, off) + scalar(3, B); };
        std::string const relu = "ite_>=[constant{f32|0},hole|f32@0,constant{f32|0},hole|f32@0]";
        std::string es = scalar(1, n) + bytes(2, scalar(1, 0)) + scalar(3, 1) + bytes(4, relu);
        std::string apply = scalar(1, 0) + scalar(2, B) + scalar(2, 0) + scalar(3, B) +
                            scalar(3, B) + bytes(4, es) + scalar(6, uint64_t(-1));
        std::string sto = scalar(1, 0) + scalar(2, 9) + scalar(3, 0);
        std::string wire = scalar(1, 1) + scalar(2, 1) +
                           bytes(4, bytes(1, los(0))) +                                   // 0
                           bytes(4, bytes(9, los(B))) +                                   // 1
                           bytes(4, bytes(4, apply) + scalar(11, 0) + scalar(11, 1)) +    // 2
                           bytes(4, bytes(6, sto + scalar(4, B) + scalar(5, B)) + scalar(11, 2)) +
                           bytes(4, bytes(7, sto + scalar(4, 2 * B) + scalar(5, B)) + scalar(11, 3));
        exec_graph_t g(km);
        expect(g.load_memgraph(wire) == 5, "memgraph: five nodes");
        expect(g.arena_bytes() == 3 * B, "memgraph: arena size");
        g.finalize(2);
        g.run(stream, arena.ptr);
        HIP_OK(hipStreamSynchronize(stream));
        arena.download(got.data());
        g.storage_read(9, slot.data(), B);
        bool ok = true;
        for (uint64_t i = 0; i != n; ++i) {
            float r = std::max(x[i], 0.0f);
            ok = ok && got[n + i] == r && got[2 * n + i] == r && slot[i] == r;
        }
        expect(ok, "memgraph from wire: apply, evict to host storage, load back");
    }

    {  // a host event loop over the exec nodes, as exec_state_t drives them
       // (src/engine/exec_state.cc:197-219): every node is launched by itself once all it
       // depends on has called back; streams and scratch come from the two pools.  The graph:
       // relu(x) -> copy (a formation) -> exp -> to_f16, and a column sum that needs scratch.
        uint64_t const n = 64 * 1024, B = n * 4;
        std::string const relu = "ite_>=[constant{f32|0},hole|f32@0,constant{f32|0},hole|f32@0]";
        einsummable_t e_relu{{n}, {{0}}, 1, relu, std::nullopt};
        einsummable_t e_exp{{n}, {{0}}, 1, "exp[hole|f32@0]", std::nullopt};
        einsummable_t e_half{{n}, {{0}}, 1, "to_f16[hole|f32@0]", std::nullopt};
        einsummable_t e_col{{256, 256}, {{1, 0}}, 1, "hole|f32@0", castable_t::add};
        auto x = random_f32(gen, n, -2, 2);
        auto build_graph = [&](exec_graph_t& g) {
            int a = g.insert_einsummable(e_relu, {{1 * B, B}, {0, B}});
            touch_t copy{{{n, n, 0, 0, n}}, std::nullopt, dtype_t::f32};
            int b = g.insert_touch(copy, -1, {2 * B, B}, {1 * B, B}, {a});
            g.insert_dummy({1 * B, B}, {b});                       // del of relu's first home
            int c = g.insert_einsummable(e_exp, {{3 * B, B}, {2 * B, B}}, {b});
            int d = g.insert_einsummable(e_half, {{4 * B, B / 2}, {3 * B, B}}, {c});
            g.insert_dummy({3 * B, B}, {d});                       // del of exp's output
            return g.insert_einsummable(e_col, {{5 * B, 1024}, {2 * B, B}}, {b});
        };
        auto run_loop = [&](exec_graph_t& g, device_buffer_t& arena, int N) {
            struct done_t {
                std::mutex              m;
                std::condition_variable cv;
                std::vector<int>        finished;
            } done;
            struct note_t {
                done_t* d;
                int     id;
            };
            std::vector<note_t> notes;
            for (int i = 0; i != N; ++i) notes.push_back({&done, i});
            std::vector<std::vector<int>> deps;
            std::vector<int>              waiting(N, 0);
            for (int i = 0; i != N; ++i) {
                deps.push_back(g.node_deps(i));
                waiting[size_t(i)] = int(deps.back().size());
            }
            workspace_pool_t ws_pool(0);
            stream_pool_t    st_pool(0, 2);
            std::vector<void*> held_ws(N, nullptr), held_st(N, nullptr);
            std::vector<int>   ready;
            for (int i = 0; i != N; ++i) {
                if (waiting[size_t(i)] == 0) ready.push_back(i);
            }
            int completed = 0;
            while (completed != N) {
                // launch what is ready while a stream is free
                while (!ready.empty()) {
                    void* st = st_pool.try_acquire();
                    if (!st) break;
                    int const id = ready.back();
                    ready.pop_back();
                    uint64_t const need = g.node_workspace(id);
                    uint64_t       got = 0;
                    held_ws[size_t(id)] = need ? ws_pool.acquire(need, &got) : nullptr;
                    held_st[size_t(id)] = st;
                    g.launch(id, st, arena.ptr, held_ws[size_t(id)], got,
                             [](void* u) {
                                 note_t* nt = static_cast<note_t*>(u);
                                 std::lock_guard<std::mutex> lk(nt->d->m);
                                 nt->d->finished.push_back(nt->id);
                                 nt->d->cv.notify_one();
                             },
                             &notes[size_t(id)]);
                }
                std::vector<int> fin;
                {
                    std::unique_lock<std::mutex> lk(done.m);
                    done.cv.wait(lk, [&] { return !done.finished.empty(); });
                    fin.swap(done.finished);
                }
                for (int id : fin) {
                    ++completed;
                    st_pool.release(held_st[size_t(id)]);
                    if (held_ws[size_t(id)]) ws_pool.release(held_ws[size_t(id)]);
                    for (int v = 0; v != N; ++v) {
                        if (std::find(deps[size_t(v)].begin(), deps[size_t(v)].end(), id) != deps[size_t(v)].end() &&
                            --waiting[size_t(v)] == 0) {
                            ready.push_back(v);
                        }
                    }
                }
            }
            HIP_OK(hipDeviceSynchronize());
            return ws_pool.blocks();
        };
        std::vector<float> host(6 * n, 7.0f);
        std::copy(x.begin(), x.end(), host.begin());
        device_buffer_t arena1(6 * B), arena2(6 * B);
        arena1.upload(host.data());
        arena2.upload(host.data());
        exec_graph_t g1(km), g2(km);
        int const col_id = build_graph(g1);
        build_graph(g2);
        expect(g2.optimize() == 2, "optimize: the copy and the exp are absorbed");
        g1.finalize(2);
        g2.finalize(2);
        expect(g1.n_launches() == 5 && g2.n_launches() == 3, "launch counts");
        int const blocks = run_loop(g1, arena1, col_id + 1);
        expect(blocks == (g1.node_workspace(col_id) ? 1 : 0), "scratch blocks in the pool");
        g2.run(stream, arena2.ptr);
        HIP_OK(hipStreamSynchronize(stream));
        std::vector<float> a1(6 * n), a2(6 * n);
        arena1.download(a1.data());
        arena2.download(a2.data());
        // against the oracle: relu, exp rounded to f16, column sums
        std::vector<float> r(n), ex(n), col(256);
        std::vector<uint16_t> hf(n);
        oracle_run(e_relu, r.data(), {x.data()});
        oracle_run(e_exp, ex.data(), {r.data()});
        oracle_run(e_half, hf.data(), {ex.data()});
        oracle_run(e_col, col.data(), {r.data()});
        bool ok = std::memcmp(&a1[2 * n], r.data(), B) == 0;
        uint16_t const* h1 = reinterpret_cast<uint16_t const*>(&a1[4 * n]);
        double          worst = 0;
        for (uint64_t i = 0; i != n; ++i) {
            double a = es_oracle_f16_to_f32(h1[i]), b = es_oracle_f16_to_f32(hf[i]);
            worst = std::max(worst, std::fabs(a - b) / std::max(std::fabs(b), 1.0));
        }
        for (int i = 0; i != 256; ++i) {
            worst = std::max(worst, std::fabs(double(a1[5 * n + i]) - col[size_t(i)]) / 256.0);
        }
        // (one f16 ulp is 2^-10 of the value: exp differs from the oracle's in the last place)
        expect(ok && worst <= 2e-3, "event loop: results against the oracle");
        // the optimised burst keeps every range it still writes
        expect(std::memcmp(&a1[2 * n], &a2[2 * n], B) == 0 &&
                   std::memcmp(&a1[4 * n], &a2[4 * n], B / 2) == 0 &&
                   std::memcmp(&a1[5 * n], &a2[5 * n], 1024) == 0,
               "optimised graph: same bytes in every range still written");

        // the entry point that allocates nothing, against the one with a workspace argument
        device_buffer_t dx(B), o1(1024), o2(1024);
        dx.upload(r.data());
        auto ws = km.build(e_col);
        device_buffer_t dws(ws.value().value());
        km(e_col, stream, o1.ptr, {dx.ptr}, std::make_tuple(dws.ptr, ws.value().value()));
        km.execute_static_workspace(e_col, stream, o2.ptr, {dx.ptr});
        HIP_OK(hipStreamSynchronize(stream));
        std::vector<float> c1(256), c2(256);
        o1.download(c1.data());
        o2.download(c2.data());
        expect(std::memcmp(c1.data(), c2.data(), 1024) == 0, "static workspace: same bits");
    }

    HIP_OK(hipStreamDestroy(stream));
    std::printf("PASS\n");
    return 0;
}
