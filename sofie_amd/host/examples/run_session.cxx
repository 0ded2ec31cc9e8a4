// Runs a generated Session: reads the input tensor(s) from raw files, calls infer(), writes the output.
// Compile with -DSOFIE_MODEL_HEADER='"x.hxx"' -DSOFIE_MODEL_NS=SOFIE_x -DSOFIE_IN_T=float -DSOFIE_OUT_T=float -DSOFIE_INPUT_MEMBER=fInput_x
// and, for a model with several inputs, -DSOFIE_NUM_INPUTS=n (then <input.bin> is a comma-separated list, one file per input
// in the order of infer()'s arguments, and there is no timing).
// For a model with several outputs add -DSOFIE_NUM_OUTPUTS=n: <output.bin> is then a comma-separated list, one file per
// output in the order of the model's output list (infer() returns a vector of vectors or a tuple of vectors), no timing.
// With -DSOFIE_NO_SESSION (a model generated with Options::kNoSession) the runner calls the free function infer() of the
// model's namespace twice and writes the second result; the weight file argument is ignored.
// With -DSOFIE_RUNTIME_BATCH (a Session generated with Options::kRuntimeBatch) the fourth argument is the batch: the
// runner calls infer(batch, input) and writes that many rows.
//   run_session <weights.dat> <input.bin> <output.bin> [timed iterations of infer_device | batch]
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <memory>
#include <sstream>
#include <string>
#include <thread>
#include <tuple>
#include <utility>
#include <vector>

#include SOFIE_MODEL_HEADER

#ifndef SOFIE_NUM_INPUTS
#define SOFIE_NUM_INPUTS 1
#endif
#ifndef SOFIE_NUM_OUTPUTS
#define SOFIE_NUM_OUTPUTS 1
#endif

static std::vector<std::string> SplitList(const std::string &list)
{
   std::vector<std::string> parts;
   size_t start = 0;
   for (size_t comma; (comma = list.find(',', start)) != std::string::npos; start = comma + 1) parts.push_back(list.substr(start, comma - start));
   parts.push_back(list.substr(start));
   return parts;
}

template <class T>
static void WriteRaw(const std::string &path, const std::vector<T> &y)
{
   std::ofstream fout(path, std::ios::binary);
   fout.write(reinterpret_cast<const char *>(y.data()), y.size() * sizeof(T));
   if (!fout) throw std::runtime_error("cannot write " + path);
}

#if SOFIE_NUM_OUTPUTS > 1
// several outputs of one type: a vector of vectors
template <class T>
static void WriteOutputs(const std::vector<std::string> &paths, const std::vector<std::vector<T>> &ys)
{
   if (ys.size() != paths.size()) throw std::runtime_error("the model returns " + std::to_string(ys.size()) + " outputs");
   for (size_t i = 0; i < ys.size(); ++i) WriteRaw(paths[i], ys[i]);
}
// outputs of different types: a tuple of vectors
template <class... V, size_t... I>
static void WriteTuple(const std::vector<std::string> &paths, const std::tuple<V...> &ys, std::index_sequence<I...>)
{
   (WriteRaw(paths[I], std::get<I>(ys)), ...);
}
template <class... V>
static void WriteOutputs(const std::vector<std::string> &paths, const std::tuple<V...> &ys)
{
   if (sizeof...(V) != paths.size()) throw std::runtime_error("the model returns " + std::to_string(sizeof...(V)) + " outputs");
   WriteTuple(paths, ys, std::index_sequence_for<V...>{});
}
#endif

static std::vector<SOFIE_IN_T> ReadRaw(const std::string &path)
{
   std::ifstream fin(path, std::ios::binary | std::ios::ate);
   if (!fin) throw std::runtime_error("cannot open input file " + path);
   const size_t bytes = fin.tellg();
   fin.seekg(0);
   std::vector<SOFIE_IN_T> x(bytes / sizeof(SOFIE_IN_T));
   fin.read(reinterpret_cast<char *>(x.data()), bytes);
   return x;
}

#if SOFIE_NUM_INPUTS > 1
template <size_t... I>
static auto InferAll(SOFIE_MODEL_NS::Session &s, std::vector<std::vector<SOFIE_IN_T>> &xs, std::index_sequence<I...>)
{
   return s.infer(xs[I].data()...);
}
#endif

int main(int argc, char **argv)
{
   if (argc < 4) {
      std::cerr << "usage: run_session <weights.dat> <input.bin> <output.bin> [iterations]\n";
      return 2;
   }
   try {
#ifdef SOFIE_NO_SESSION
      {
         std::vector<SOFIE_IN_T> x = ReadRaw(argv[2]);
         SOFIE_MODEL_NS::infer(x.data());
         WriteRaw(argv[3], SOFIE_MODEL_NS::infer(x.data()));
         return 0;
      }
#endif
      SOFIE_MODEL_NS::Session s(argv[1]);
#if SOFIE_NUM_INPUTS > 1
      std::vector<std::vector<SOFIE_IN_T>> xs;
      {
         std::string list = argv[2];
         size_t start = 0;
         for (size_t comma; (comma = list.find(',', start)) != std::string::npos; start = comma + 1)
            xs.push_back(ReadRaw(list.substr(start, comma - start)));
         xs.push_back(ReadRaw(list.substr(start)));
         if (xs.size() != SOFIE_NUM_INPUTS) throw std::runtime_error("the model takes " + std::to_string(SOFIE_NUM_INPUTS) + " input files");
      }
      auto y = InferAll(s, xs, std::make_index_sequence<SOFIE_NUM_INPUTS>{});
#if SOFIE_NUM_OUTPUTS > 1
      WriteOutputs(SplitList(argv[3]), y);
#else
      WriteRaw(argv[3], y);
#endif
#else
      std::vector<SOFIE_IN_T> x = ReadRaw(argv[2]);
#if SOFIE_NUM_OUTPUTS > 1
      WriteOutputs(SplitList(argv[3]), s.infer(x.data()));
      // the device-pointer form returns the same tensors' device addresses, in the same order
      auto dev = s.infer_device(s.SOFIE_INPUT_MEMBER);
      s.sync();
      static_assert(std::tuple_size<decltype(dev)>::value == SOFIE_NUM_OUTPUTS, "one device address per output");
#elif defined(SOFIE_RUNTIME_BATCH)
      std::vector<SOFIE_OUT_T> y = argc > 4 ? s.infer((size_t)std::atoi(argv[4]), x.data()) : s.infer(x.data());
      std::ofstream fout(argv[3], std::ios::binary);
      fout.write(reinterpret_cast<const char *>(y.data()), y.size() * sizeof(SOFIE_OUT_T));
      const int iters = 0;
#else
      std::vector<SOFIE_OUT_T> y = s.infer(x.data());
      std::ofstream fout(argv[3], std::ios::binary);
      fout.write(reinterpret_cast<const char *>(y.data()), y.size() * sizeof(SOFIE_OUT_T));
      const int iters = argc > 4 ? std::atoi(argv[4]) : 0;
#endif
#if SOFIE_NUM_OUTPUTS == 1
      if (iters > 0) {
         // device-resident timing: the input stays in the Session's device buffer
         // as many untimed runs as timed ones first: the device leaves its idle clocks over some tens of milliseconds
         for (int i = 0; i < (iters > 3 ? iters : 3); ++i) s.infer_device(s.SOFIE_INPUT_MEMBER);
         s.sync();
         float ms = 0;
         sofie_hip_timer_start(s.fCtx);
         for (int i = 0; i < iters; ++i) s.infer_device(s.SOFIE_INPUT_MEMBER);
         sofie_hip_timer_stop(s.fCtx, &ms);
         auto t0 = std::chrono::steady_clock::now();
         for (int i = 0; i < iters; ++i) y = s.infer(x.data());
         const double host_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
         // the same calls on the Session's page-locked input buffer: the upload runs at the rate of the link
         SOFIE_IN_T *pinned = s.SOFIE_PINNED_INPUT();
         std::memcpy(pinned, x.data(), x.size() * sizeof(SOFIE_IN_T));
         std::vector<SOFIE_OUT_T> yp = s.infer(pinned);
         bool pinned_same = yp.size() == y.size() && std::memcmp(yp.data(), y.data(), y.size() * sizeof(SOFIE_OUT_T)) == 0;
         t0 = std::chrono::steady_clock::now();
         for (int i = 0; i < iters; ++i) yp = s.infer(pinned);
         const double pinned_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
         // the same sequence replayed from a HIP graph: outputs must not change, timing of back-to-back replays
         bool same = true;
         float gms = 0;
         {
            s.use_graph(true);
            std::vector<SOFIE_OUT_T> yg = s.infer(x.data());
            same = yg.size() == y.size();
            for (int rep = 0; rep < 3 && same; ++rep) {
               s.infer_device(s.SOFIE_INPUT_MEMBER);   // eager work and a synchronisation between replays
               s.sync();
               yg = s.infer(x.data());
               for (size_t i = 0; i < y.size() && same; ++i) same = std::memcmp(&yg[i], &y[i], sizeof(SOFIE_OUT_T)) == 0;
            }
            s.sync();
            sofie_hip_timer_start(s.fCtx);
            for (int i = 0; i < iters; ++i) s.run_own_input();
            sofie_hip_timer_stop(s.fCtx, &gms);
         }
         // Several Sessions in flight (a context and a stream each, a host thread each, as the slots of a SofieFunctor
         // run; two unless SOFIE_RUN_SESSIONS says otherwise): the device overlaps the start of one Session's kernels with
         // the others'. Wall time over all of them, per batch.
         double pair_ms = 0;
         bool pair_same = true;
         int nsess = 2;
         if (const char *e = std::getenv("SOFIE_RUN_SESSIONS")) nsess = std::atoi(e);
         if (nsess >= 2 && !std::getenv("SOFIE_RUN_NO_PAIR")) {
            s.use_graph(false);
            std::vector<std::unique_ptr<SOFIE_MODEL_NS::Session>> others;
            for (int k = 1; k < nsess; ++k) {
               others.emplace_back(new SOFIE_MODEL_NS::Session(argv[1]));
               std::vector<SOFIE_OUT_T> y2 = others.back()->infer(x.data());   // leaves the input in that Session's device buffer
               pair_same = pair_same && y2.size() == y.size() && std::memcmp(y2.data(), y.data(), y.size() * sizeof(SOFIE_OUT_T)) == 0;
            }
            // every Session's last result is read back after the runs in flight and compared with the serial one
            std::vector<const SOFIE_OUT_T *> results(nsess, nullptr);
            auto run = [iters, &results](SOFIE_MODEL_NS::Session *sess, int slot) {
               for (int i = 0; i < iters; ++i) results[slot] = sess->infer_device(sess->SOFIE_INPUT_MEMBER);
               sess->sync();
            };
            auto all_at_once = [&]() {
               std::vector<std::thread> workers;
               for (size_t k = 0; k < others.size(); ++k) workers.emplace_back(run, others[k].get(), (int)k + 1);
               run(&s, 0);
               for (auto &w : workers) w.join();
            };
            all_at_once();     // untimed
            t0 = std::chrono::steady_clock::now();
            all_at_once();
            pair_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() / ((double)nsess * iters);
            for (int k = 0; k < nsess; ++k) {
               SOFIE_MODEL_NS::Session *sess = k == 0 ? &s : others[k - 1].get();
               std::vector<SOFIE_OUT_T> yk(y.size());
               const bool read = results[k] && sofie_hip_download(sess->fCtx, yk.data(), results[k], yk.size() * sizeof(SOFIE_OUT_T)) == 0;
               pair_same = pair_same && read && std::memcmp(yk.data(), y.data(), y.size() * sizeof(SOFIE_OUT_T)) == 0;
            }
         }
         // Per launch: an event behind every kernel of the sequence (sofie_hip_trace_begin / _end), over up to 200 runs
         // back to back; a launch's time runs from the end of the launch before it, so the entries of a run add up to
         // the run. Averaged by position in the run.
         std::string kernels = "[";
         {
            const int passes = iters < 200 ? iters : 200;
            std::vector<char> text(1 << 20);
            int seen = 0;
            if (sofie_hip_trace_begin(s.fCtx) == 0) {
               for (int i = 0; i < passes; ++i) s.infer_device(s.SOFIE_INPUT_MEMBER);
               if (sofie_hip_trace_end(s.fCtx, text.data(), text.size(), &seen) == 0 && seen > 0 && seen % passes == 0 &&
                   seen <= SOFIE_HIP_TRACE_MAX) {
                  const int per = seen / passes;
                  std::vector<std::string> names(per);
                  std::vector<double> sum(per, 0.0);
                  std::istringstream lines(text.data());
                  std::string name;
                  double us = 0;
                  int k = 0;
                  for (; lines >> name >> us; ++k) {
                     names[k % per] = name;
                     sum[k % per] += us;
                  }
                  if (k == seen) {
                     for (int j = 0; j < per; ++j) {
                        char item[256];
                        std::snprintf(item, sizeof(item), "%s{\"kernel\": \"%s\", \"us\": %.3f}", j ? ", " : "", names[j].c_str(), sum[j] / passes);
                        kernels += item;
                     }
                  }
               }
            }
         }
         kernels += "]";
         std::printf("{\"device_ms\": %.6f, \"host_ms\": %.6f, \"host_pinned_ms\": %.6f, \"pinned_matches\": %s, \"graph_ms\": %.6f, "
                     "\"graph_matches\": %s, \"sessions_in_flight\": %d, \"two_sessions_ms_per_batch\": %.6f, \"two_sessions_match\": %s, "
                     "\"iters\": %d, \"kernels\": %s}\n",
                     ms / iters, host_ms / iters, pinned_ms / iters, pinned_same ? "true" : "false", gms / iters,
                     same ? "true" : "false", nsess, pair_ms, pair_same ? "true" : "false", iters, kernels.c_str());
      }
#endif
#endif
   } catch (const std::exception &e) {
      std::cerr << "run_session: " << e.what() << "\n";
      return 1;
   }
   return 0;
}
