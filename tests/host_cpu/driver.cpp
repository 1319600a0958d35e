// Test driver of the CPU build of libtm_hip's host logic: reads a program of
// C-ABI calls from stdin, one per line, runs it against the stand-in runtime and
// the recording launchers, and prints one JSON object per line: what each
// command returned, every launch the library issued, and the counters asked for.
// Built by tests/test_host_logic_cpu.py with -fsanitize=address,undefined.
//
// Commands (buffers and steps are named; sizes in bytes unless said otherwise):
//   ctx NAME | use NAME | destroy NAME
//   buf NAME BYTES [private] | free NAME | seal NAME ROWS COLS | zero NAME OFF LEN
//   upload NAME OFF LEN | download NAME OFF LEN
//   gemv W X Y ROWS COLS | gemm W X Y ROWS COLS BATCH XOFF YOFF | mma ... | mma_noalloc ...
//   f16gemm W X Y ROWS COLS BATCH XOFF YOFF
//   quant X XQ COLS BATCH XOFF | i8 W XQ Y ROWS COLS BATCH YOFF | i8fma ...
//   rmsnorm X WEIGHT Y ROWS COLS | silu G U OUT N | gelu G U OUT N | axpy A Y ALPHA N
//   scale X Y FACTOR N | copy SRC SOFF DST DOFF N | argmax X N PARTIAL OUT INDEX
//   checksum SRC SOFF N PARTIAL | row W OUT ROW COLS OUTOFF
//   begin | end | abort | fence | record STEP | run STEP | stepfree STEP
//   download_after NAME OFF LEN COMPLETED_TARGET | profile 0|1 | commitlog 0|1 | measure
//   advance N | eager 0|1 | failmalloc N | stats | mark TEXT
// A command prefixed with "!" is expected to fail; its code is reported either way.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <map>
#include <sstream>
#include <string>
#include <vector>

#include "recorder.hpp"
#include "tm_hip.h"

namespace {

struct Named {
    tm_hip_ctx *ctx;
    tm_hip_buffer *buf;
};
std::map<std::string, tm_hip_ctx *> contexts;
std::map<std::string, Named> buffers;
std::map<std::string, std::pair<tm_hip_ctx *, tm_hip_step *>> steps;
tm_hip_ctx *cur = nullptr;
char err[1024];

void flush_launches() {
    for (const std::string &l : rec::log) {
        printf("%s\n", l.c_str());
    }
    rec::log.clear();
}

tm_hip_buffer *B(const std::string &name) {
    if (name == "null") {
        return nullptr;
    }
    auto it = buffers.find(name);
    if (it == buffers.end()) {
        fprintf(stderr, "driver: no buffer named %s\n", name.c_str());
        exit(2);
    }
    return it->second.buf;
}

// Buffers must be freed before their context goes (native/metal/tm_metal.h:56):
// the handles the program still holds are freed here; steps it never freed and a
// group it left open are the library's to dispose of.
void destroy_context(tm_hip_ctx *c) {
    for (auto it = buffers.begin(); it != buffers.end();) {
        if (it->second.ctx == c) {
            tm_hip_buffer_free(c, it->second.buf);
            it = buffers.erase(it);
        } else {
            ++it;
        }
    }
    for (auto it = steps.begin(); it != steps.end();) {
        it = it->second.first == c ? steps.erase(it) : std::next(it);
    }
    tm_hip_destroy(c);
}

std::string json_escape(const char *s) {
    std::string o;
    for (; *s; ++s) {
        if (*s == '"' || *s == '\\') {
            o += '\\';
        }
        o += *s >= 32 ? *s : ' ';
    }
    return o;
}

} // namespace

// The launchers name allocations by their device address, the driver holds opaque
// handles: it tells allocations apart by their order of allocation in the
// stand-in runtime (tm_hip_buffer_new and tm_hip_q8_0_pack make exactly one each).
static std::map<uint64_t, std::string> names_by_serial;
static std::string name_of(const void *p) {
    const uint64_t serial = fake::serial_of(p);
    auto it = names_by_serial.find(serial);
    if (it != names_by_serial.end()) {
        return it->second;
    }
    return "@" + std::to_string(serial);
}

int main() {
    rec::name_of = name_of;
    std::string line;
    long lineno = 0;
    while (std::getline(std::cin, line)) {
        ++lineno;
        if (line.empty() || line[0] == '#') {
            continue;
        }
        bool expect_fail = false;
        if (line[0] == '!') {
            expect_fail = true;
            line = line.substr(1);
        }
        std::istringstream in(line);
        std::string cmd;
        in >> cmd;
        int rc = 0;
        bool is_call = true;
        err[0] = '\0';
        auto u32 = [&]() {
            unsigned long long v = 0;
            in >> v;
            return (uint32_t)v;
        };
        auto sz = [&]() {
            unsigned long long v = 0;
            in >> v;
            return (size_t)v;
        };
        auto str = [&]() {
            std::string s;
            in >> s;
            return s;
        };
        if (cmd == "ctx") {
            const std::string name = str();
            tm_hip_ctx *c = tm_hip_create(err, sizeof err);
            rc = c != nullptr ? 0 : -1;
            if (c != nullptr) {
                contexts[name] = c;
                cur = c;
            }
        } else if (cmd == "use") {
            cur = contexts.at(str());
            is_call = false;
        } else if (cmd == "destroy") {
            const std::string name = str();
            tm_hip_ctx *c = contexts.at(name);
            destroy_context(c);
            contexts.erase(name);
            if (cur == c) {
                cur = nullptr;
            }
        } else if (cmd == "buf") {
            const std::string name = str();
            const size_t bytes = sz();
            std::string flag;
            in >> flag;
            const uint64_t before = fake::counters().total_allocs;
            tm_hip_buffer *b = tm_hip_buffer_new(cur, bytes, flag == "private" ? 0 : 1, err, sizeof err);
            rc = b != nullptr ? 0 : -1;
            if (b != nullptr) {
                buffers[name] = Named{cur, b};
                if (fake::counters().total_allocs != before + 1) {
                    fprintf(stderr, "driver: buffer_new made %llu device allocations\n",
                            (unsigned long long)(fake::counters().total_allocs - before));
                    return 2;
                }
                names_by_serial[before + 1] = name;
            }
        } else if (cmd == "free") {
            const std::string name = str();
            auto it = buffers.find(name);
            if (it == buffers.end()) {
                fprintf(stderr, "driver: free of unknown buffer %s\n", name.c_str());
                return 2;
            }
            tm_hip_buffer_free(it->second.ctx, it->second.buf);
            buffers.erase(it);
        } else if (cmd == "seal") {
            const std::string name = str();
            tm_hip_buffer *w = B(name);
            const uint32_t rows = u32(), cols = u32();
            const uint64_t before = fake::counters().total_allocs;
            rc = tm_hip_q8_0_pack(cur, w, rows, cols, err, sizeof err);
            if (rc == 0) { // the handle now names a fresh, sealed allocation
                for (auto &kv : names_by_serial) {
                    if (kv.second == name) {
                        kv.second = name + ".raw";
                    }
                }
                names_by_serial[before + 1] = name;
            }
        } else if (cmd == "zero") {
            tm_hip_buffer *b = B(str());
            const size_t off = sz(), len = sz();
            rc = tm_hip_buffer_zero(cur, b, off, len, err, sizeof err);
        } else if (cmd == "upload" || cmd == "download") {
            tm_hip_buffer *b = B(str());
            const size_t off = sz(), len = sz();
            std::vector<uint8_t> host(len ? len : 1, 0x5a);
            rc = cmd == "upload" ? tm_hip_upload(cur, b, off, host.data(), len, err, sizeof err)
                                 : tm_hip_download(cur, b, off, host.data(), len, err, sizeof err);
        } else if (cmd == "gemv") {
            tm_hip_buffer *w = B(str()), *x = B(str()), *y = B(str());
            const uint32_t rows = u32(), cols = u32();
            rc = tm_hip_q8_0_gemv(cur, w, x, y, rows, cols, err, sizeof err);
        } else if (cmd == "gemm" || cmd == "mma" || cmd == "mma_noalloc" || cmd == "f16gemm") {
            tm_hip_buffer *w = B(str()), *x = B(str()), *y = B(str());
            const uint32_t rows = u32(), cols = u32(), batch = u32(), xoff = u32(), yoff = u32();
            auto fn = cmd == "gemm"          ? tm_hip_q8_0_gemm
                      : cmd == "mma"         ? tm_hip_q8_0_gemm_mma
                      : cmd == "mma_noalloc" ? tm_hip_q8_0_gemm_mma_noalloc
                                             : tm_hip_f16_gemm;
            rc = fn(cur, w, x, y, rows, cols, batch, xoff, yoff, err, sizeof err);
        } else if (cmd == "quant") {
            tm_hip_buffer *x = B(str()), *xq = B(str());
            const uint32_t cols = u32(), batch = u32(), xoff = u32();
            rc = tm_hip_q8_0_quantize_act(cur, x, xq, cols, batch, xoff, err, sizeof err);
        } else if (cmd == "i8" || cmd == "i8fma") {
            tm_hip_buffer *w = B(str()), *xq = B(str()), *y = B(str());
            const uint32_t rows = u32(), cols = u32(), batch = u32(), yoff = u32();
            rc = cmd == "i8" ? tm_hip_q8_0_gemm_i8(cur, w, xq, y, nullptr, rows, cols, batch, yoff, err, sizeof err)
                             : tm_hip_q8_0_gemm_i8_fma(cur, w, xq, y, rows, cols, batch, yoff, err, sizeof err);
        } else if (cmd == "rmsnorm") {
            tm_hip_buffer *x = B(str()), *w = B(str()), *y = B(str());
            const uint32_t rows = u32(), cols = u32();
            rc = tm_hip_rmsnorm_f32(cur, x, w, y, rows, cols, 1e-6f, err, sizeof err);
        } else if (cmd == "silu" || cmd == "gelu") {
            tm_hip_buffer *g = B(str()), *u = B(str()), *o = B(str());
            const uint32_t n = u32();
            rc = cmd == "silu" ? tm_hip_silu_mul_f32(cur, g, u, o, n, err, sizeof err)
                               : tm_hip_gelu_tanh_mul_f32(cur, g, u, o, n, err, sizeof err);
        } else if (cmd == "axpy" || cmd == "scale") {
            tm_hip_buffer *a = B(str()), *y = B(str());
            float alpha = 0.0f;
            in >> alpha;
            const uint32_t n = u32();
            rc = cmd == "axpy" ? tm_hip_f32_axpy(cur, a, y, alpha, n, err, sizeof err)
                               : tm_hip_f32_scale(cur, a, y, alpha, n, err, sizeof err);
        } else if (cmd == "copy") {
            tm_hip_buffer *s = B(str());
            const uint32_t soff = u32();
            tm_hip_buffer *d = B(str());
            const uint32_t doff = u32(), n = u32();
            rc = tm_hip_copy_f32(cur, s, soff, d, doff, n, err, sizeof err);
        } else if (cmd == "argmax") {
            tm_hip_buffer *x = B(str());
            const uint32_t n = u32();
            tm_hip_buffer *part = B(str()), *out = B(str());
            const uint32_t index = u32();
            rc = tm_hip_argmax_f32(cur, x, n, part, out, index, err, sizeof err);
        } else if (cmd == "checksum") {
            tm_hip_buffer *s = B(str());
            const uint32_t soff = u32(), n = u32();
            tm_hip_buffer *part = B(str());
            rc = tm_hip_xor_checksum_u32(cur, s, soff, n, part, err, sizeof err);
        } else if (cmd == "row") {
            tm_hip_buffer *w = B(str()), *out = B(str());
            const uint32_t row = u32(), cols = u32(), off = u32();
            rc = tm_hip_q8_0_row_f32(cur, w, out, row, cols, off, err, sizeof err);
        } else if (cmd == "begin") {
            rc = tm_hip_begin_group(cur, err, sizeof err);
        } else if (cmd == "end") {
            rc = tm_hip_end_group(cur, err, sizeof err);
        } else if (cmd == "abort") {
            rc = tm_hip_abort_group(cur, err, sizeof err);
        } else if (cmd == "fence") {
            rc = tm_hip_fence(cur, err, sizeof err);
        } else if (cmd == "record") {
            const std::string name = str();
            tm_hip_step *step = nullptr;
            rc = tm_hip_end_group_recorded(cur, &step, err, sizeof err);
            if (rc == 0) {
                steps[name] = {cur, step};
            }
        } else if (cmd == "run") {
            rc = tm_hip_step_run(cur, steps.at(str()).second, err, sizeof err);
        } else if (cmd == "stepfree") {
            const std::string name = str();
            tm_hip_step_free(steps.at(name).first, steps.at(name).second);
            steps.erase(name);
        } else if (cmd == "download_after") {
            tm_hip_buffer *b = B(str());
            const size_t off = sz(), len = sz();
            const uint64_t target = (uint64_t)sz();
            std::vector<uint8_t> host(len ? len : 1, 0x5a);
            rc = tm_hip_download_after(cur, b, off, host.data(), len, target, err, sizeof err);
        } else if (cmd == "profile") {
            rc = tm_hip_profile_set(cur, (int)u32());
        } else if (cmd == "commitlog") {
            rc = tm_hip_commit_log_set(cur, (int)u32());
        } else if (cmd == "measure") {
            // every entry point that reads the commits' events
            is_call = false;
            flush_launches();
            const double ms = tm_hip_last_gpu_ms(cur);
            const uint64_t total = tm_hip_gpu_nanos_total(cur);
            std::vector<uint64_t> log(TM_HIP_COMMIT_LOG_CAP);
            const size_t logged = tm_hip_commit_log_read(cur, log.data(), log.size());
            uint32_t slots = 0;
            uint64_t count_sum = 0;
            char name[64];
            uint64_t nanos = 0, count = 0;
            while (tm_hip_profile_read(cur, slots, name, sizeof name, &nanos, &count) == 1) {
                ++slots;
                count_sum += count;
            }
            printf("{\"k\":\"measure\",\"last_ms\":%g,\"total_ns\":%llu,\"logged\":%zu,"
                   "\"profile_slots\":%u,\"profile_count\":%llu}\n",
                   ms, (unsigned long long)total, logged, slots, (unsigned long long)count_sum);
            continue;
        } else if (cmd == "advance") {
            fake::advance_all(sz());
            is_call = false;
        } else if (cmd == "eager") {
            fake::set_eager(u32() != 0);
            is_call = false;
        } else if (cmd == "failmalloc") {
            fake::fail_malloc_after(sz());
            is_call = false;
        } else if (cmd == "mark") {
            std::string rest;
            std::getline(in, rest);
            flush_launches();
            printf("{\"k\":\"mark\",\"text\":\"%s\"}\n", json_escape(rest.c_str()).c_str());
            continue;
        } else if (cmd == "stats") {
            flush_launches();
            // (the library's own figures first: asking for them retires what has completed)
            unsigned long long lib[5] = {0, 0, 0, 0, 0};
            if (cur != nullptr) {
                lib[3] = tm_hip_completed_dispatches(cur);
                lib[0] = tm_hip_allocated_bytes(cur);
                lib[1] = tm_hip_in_flight_bytes(cur);
                lib[2] = tm_hip_committed_dispatches(cur);
                lib[4] = tm_hip_kernel_launches(cur);
            }
            const fake::Counters c = fake::counters();
            printf("{\"k\":\"stats\",\"live_allocs\":%llu,\"live_bytes\":%llu,\"live_streams\":%llu,"
                   "\"live_events\":%llu,\"live_graphs\":%llu,\"live_execs\":%llu,\"enqueued\":%llu,"
                   "\"graph_launches\":%llu",
                   (unsigned long long)c.live_allocs, (unsigned long long)c.live_bytes,
                   (unsigned long long)c.live_streams, (unsigned long long)c.live_events,
                   (unsigned long long)c.live_graphs, (unsigned long long)c.live_execs,
                   (unsigned long long)c.enqueued, (unsigned long long)c.graph_launches);
            if (cur != nullptr) {
                printf(",\"allocated\":%llu,\"in_flight\":%llu,\"committed\":%llu,\"completed\":%llu,"
                       "\"launches\":%llu", lib[0], lib[1], lib[2], lib[3], lib[4]);
            }
            printf("}\n");
            continue;
        } else {
            fprintf(stderr, "driver: line %ld: unknown command %s\n", lineno, cmd.c_str());
            return 2;
        }
        flush_launches();
        if (is_call) {
            if ((rc != 0) != expect_fail) {
                fprintf(stderr, "driver: line %ld `%s` returned %d (%s), expected %s\n", lineno,
                        line.c_str(), rc, err, expect_fail ? "a refusal" : "success");
                return 3;
            }
            printf("{\"k\":\"ret\",\"cmd\":\"%s\",\"rc\":%d,\"err\":\"%s\"}\n", cmd.c_str(), rc,
                   json_escape(err).c_str());
        }
    }
    flush_launches();
    // whatever the program left open goes with its context
    for (auto &c : contexts) {
        destroy_context(c.second);
    }
    const fake::Counters c = fake::counters();
    printf("{\"k\":\"exit\",\"live_allocs\":%llu,\"live_streams\":%llu,\"live_events\":%llu,"
           "\"live_graphs\":%llu,\"live_execs\":%llu}\n",
           (unsigned long long)c.live_allocs, (unsigned long long)c.live_streams,
           (unsigned long long)c.live_events, (unsigned long long)c.live_graphs,
           (unsigned long long)c.live_execs);
    return 0;
}
