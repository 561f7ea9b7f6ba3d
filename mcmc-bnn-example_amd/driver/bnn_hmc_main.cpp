// Host driver of the MI355X HMC sampler: the three phases of the reference's mcmc::main_loop
// (include/mcmc/main.h:117-308) -- init, run N samples, dump the chain -- on top of the C ABI in
// include/bnn_hmc.h.  Plain C++, no GPU code here.
//
//   bnn_hmc_main [--windows W] [--chains C] [--samples S] [--burn-in B] [--leapfrog L] [--rows N]
//                [--lik student_t|gaussian] [--layer mfma|ffma] [--cus-per-chain G] [--wgs-per-cu K]
//                [--seed S] [--data FILE] [--dump FILE] [--features D0 --hidden D1]   (22 40 or 64 128)
//
// --dump FILE writes the kept samples of every chain as a NumPy array file (format 1.0, little-endian
// float32, shape (chains, samples, parameters), chain = window * chains_per_window + chain of the
// window) and FILE.json beside it with what a reader needs to interpret it: shapes, layer sizes,
// model and sampler constants, seed, and per chain the final step size and the accepted transitions.
//
// Without --data every window is filled with the synthetic recipe (features ~ N(0,1), targets from
// a random teacher MLP plus noise).  With --data the reference's text format is read
// (include/mcmc/io.h:43-86) into window 0 and the features are scaled by 0.001 (main.h:162-164).
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "bnn_hmc.h"

namespace {

struct Options {
  int windows = 1, chains = 1, samples = 800, burn_in = 100, leapfrog = 1000, rows = 58368;
  int features = 22, hidden = 40;
  int lik = BNNHMC_LIK_STUDENT_T, layer = BNNHMC_LAYER_MFMA, cus_per_chain = 0, wgs_per_cu = 0;
  unsigned seed = 0;
  std::string data, dump;
};

void die(const char* what) {
  std::fprintf(stderr, "error: %s: %s\n", what, bnnhmc_last_error());
  std::exit(1);
}
#define CHECK(call)            \
  do {                         \
    if ((call) != BNNHMC_OK) die(#call); \
  } while (0)

bool parse(int argc, char** argv, Options& o) {
  for (int i = 1; i < argc; ++i) {
    std::string a = argv[i];
    auto next = [&]() -> const char* { return i + 1 < argc ? argv[++i] : ""; };
    if (a == "--windows") o.windows = std::atoi(next());
    else if (a == "--chains") o.chains = std::atoi(next());
    else if (a == "--samples") o.samples = std::atoi(next());
    else if (a == "--burn-in") o.burn_in = std::atoi(next());
    else if (a == "--leapfrog") o.leapfrog = std::atoi(next());
    else if (a == "--rows") o.rows = std::atoi(next());
    else if (a == "--features") o.features = std::atoi(next());
    else if (a == "--hidden") o.hidden = std::atoi(next());
    else if (a == "--seed") o.seed = (unsigned)std::strtoul(next(), nullptr, 10);
    else if (a == "--cus-per-chain") o.cus_per_chain = std::atoi(next());
    else if (a == "--wgs-per-cu") o.wgs_per_cu = std::atoi(next());
    else if (a == "--lik") o.lik = std::string(next()) == "gaussian" ? BNNHMC_LIK_GAUSSIAN : BNNHMC_LIK_STUDENT_T;
    else if (a == "--layer") o.layer = std::string(next()) == "ffma" ? BNNHMC_LAYER_FFMA : BNNHMC_LAYER_MFMA;
    else if (a == "--data") o.data = next();
    else if (a == "--dump") o.dump = next();
    else {
      std::fprintf(stderr, "unknown option %s\n", a.c_str());
      return false;
    }
  }
  return true;
}

// shape / min / max / mean summary the reference prints for a matrix (utils_matrix.h:160-178)
void print_stats(const char* name, const float* d, size_t rows, size_t cols) {
  float mn = INFINITY, mx = -INFINITY, mean = 0.0f;
  const size_t n = rows * cols;
  for (size_t i = 0; i < n; ++i) {
    mean += d[i] / (float)n;
    if (d[i] > mx) mx = d[i];
    if (d[i] < mn) mn = d[i];
  }
  std::printf("%s: Shape: %zu x %zu, word: 4, min: %g, max: %g, mean: %g\n", name, rows, cols, mn, mx, mean);
}

// header of a NumPy array file, format 1.0: magic, version, little-endian header length, a Python
// dict literal padded with spaces so that the data starts at a multiple of 64 bytes
void write_npy_header(FILE* f, int chains, int samples, int params) {
  char dict[192];
  const int len = std::snprintf(dict, sizeof(dict), "{'descr': '<f4', 'fortran_order': False, 'shape': (%d, %d, %d), }",
                                chains, samples, params);
  const int unpadded = 10 + len + 1;  // magic 6 + version 2 + length 2 + dict + newline
  const int pad = (64 - unpadded % 64) % 64;
  const unsigned short hlen = (unsigned short)(len + pad + 1);
  const unsigned char pre[10] = {0x93, 'N', 'U', 'M', 'P', 'Y', 1, 0, (unsigned char)(hlen & 0xff),
                                 (unsigned char)(hlen >> 8)};
  std::fwrite(pre, 1, sizeof(pre), f);
  std::fwrite(dict, 1, (size_t)len, f);
  for (int i = 0; i < pad; ++i) std::fputc(' ', f);
  std::fputc('\n', f);
}

}  // namespace

int main(int argc, char** argv) {
  Options o;
  if (!parse(argc, argv, o)) return 2;

  // ------------------------------------------------------------------ init (main.h:120-202)
  bnnhmc_model model;
  bnnhmc_default_model(&model);
  model.n = o.rows;
  model.d0 = o.features;
  model.d1 = o.hidden;
  model.lik_kind = o.lik;
  if (o.lik == BNNHMC_LIK_GAUSSIAN) {  // the benchmark configs: sigma 0.01, prior N(0, 0.1^2)
    model.lik_scale = 0.01;
    model.prior_scale = 0.1;
  }
  bnnhmc_hmc hmc;
  bnnhmc_default_hmc(&hmc);
  hmc.n_samples = o.samples;
  hmc.burn_in = o.burn_in;
  hmc.adapt_steps = o.burn_in;
  hmc.leapfrog_steps = o.leapfrog;
  hmc.seed = o.seed;
  bnnhmc_launch launch;
  bnnhmc_default_launch(&launch);
  launch.layer = o.layer;
  if (o.cus_per_chain > 0) launch.cus_per_chain = o.cus_per_chain;
  if (o.wgs_per_cu > 0) launch.wgs_per_cu = o.wgs_per_cu;

  int n_dev = 0, cus = 0;
  char arch[64];
  CHECK(bnnhmc_device_info(&n_dev, &cus, arch, sizeof(arch)));
  char groups[64];
  if (launch.cus_per_chain > 0) std::snprintf(groups, sizeof(groups), "%d workgroups per chain", launch.cus_per_chain);
  else std::snprintf(groups, sizeof(groups), "workgroups per chain chosen by the library");
  std::printf("Device 0: %s, %d compute units. %d window(s) x %d chain(s), %s, %s layer.\n", arch, cus,
              o.windows, o.chains, groups, o.layer == BNNHMC_LAYER_FFMA ? "FFMA" : "MFMA");

  bnnhmc_sampler* s = nullptr;
  CHECK(bnnhmc_create(&model, &hmc, &launch, o.windows, o.chains, &s));
  const int P = bnnhmc_num_params(model.d0, model.d1);
  if (!o.data.empty()) {
    std::vector<float> x((size_t)model.n * model.d0), y(model.n);
    std::printf("Reading dataset...\n");
    CHECK(bnnhmc_read_reference_data(o.data.c_str(), model.n, model.d0, 149, 2, x.data(), y.data()));
    std::printf("Dataset read successfully\n");
    print_stats("Data", x.data(), model.n, model.d0);
    print_stats("Labels", y.data(), model.n, 1);
    for (float& v : x) v *= 0.001f;  // main.h:162-164
    for (int w = 0; w < o.windows; ++w) CHECK(bnnhmc_set_window_data(s, w, x.data(), y.data()));
  } else {
    for (int w = 0; w < o.windows; ++w) CHECK(bnnhmc_generate_window(s, w, 0.1f, 0.01f, nullptr));
    std::vector<float> x((size_t)model.n * model.d0), y(model.n);
    CHECK(bnnhmc_get_window_data(s, 0, x.data(), y.data()));
    print_stats("Data", x.data(), model.n, model.d0);
    print_stats("Labels", y.data(), model.n, 1);
  }

  const auto t_start = std::chrono::high_resolution_clock::now();  // main.h:187-189
  CHECK(bnnhmc_init_chains(s, nullptr));

  // ------------------------------------------------------------------ run (main.h:204-287)
  // calls of 100 transitions (a progress dot each): inside one call, chains that take turns on the device
  // (more windows than fit at once) do so on launches that fill it, and only what is left at the end of a
  // call runs in narrower ones, so long calls cost less than short ones
  const int total = hmc.burn_in + hmc.n_samples, every = 100;
  for (int done = 0; done < total; done += every) {
    CHECK(bnnhmc_run(s, std::min(every, total - done)));
    std::printf(".");
    std::fflush(stdout);
  }
  std::printf("\n");
  const auto t_end = std::chrono::high_resolution_clock::now();  // main.h:293

  // ------------------------------------------------------------------ dump (main.h:295-307)
  std::vector<float> samples((size_t)hmc.n_samples * P);
  const int n_chains = o.windows * o.chains;
  int stored_all = 0;
  CHECK(bnnhmc_get_samples(s, 0, nullptr, &stored_all));
  FILE* out = nullptr;
  if (!o.dump.empty()) {
    out = std::fopen(o.dump.c_str(), "wb");
    if (!out) {
      std::fprintf(stderr, "error: cannot open %s for writing\n", o.dump.c_str());
      return 1;
    }
    write_npy_header(out, n_chains, stored_all, P);
  }
  for (int c = 0; c < n_chains; ++c) {
    int stored = 0;
    CHECK(bnnhmc_get_samples(s, c, samples.data(), &stored));
    if (c == 0) print_stats("Final samples", samples.data(), stored, P);
    if (out) std::fwrite(samples.data(), sizeof(float), (size_t)stored * P, out);
  }
  if (out) {
    std::fclose(out);
    const std::string meta = o.dump + ".json";
    FILE* mj = std::fopen(meta.c_str(), "w");
    if (!mj) {
      std::fprintf(stderr, "error: cannot open %s for writing\n", meta.c_str());
      return 1;
    }
    std::fprintf(mj,
                 "{\n \"format\": \"npy float32 little-endian, C order\",\n \"shape\": [%d, %d, %d],\n"
                 " \"axes\": [\"chain = window * chains_per_window + chain of the window\", \"kept sample\", "
                 "\"parameter: W1[k * hidden + c] | b1[c] | w2[c] | b2\"],\n"
                 " \"windows\": %d,\n \"chains_per_window\": %d,\n \"features\": %d,\n \"hidden\": %d,\n"
                 " \"rows\": %d,\n \"parameters\": %d,\n \"likelihood\": \"%s\",\n \"lik_scale\": %.17g,\n"
                 " \"lik_df\": %.17g,\n \"prior_scale\": %.17g,\n \"leapfrog_steps\": %d,\n \"burn_in\": %d,\n"
                 " \"adapt_steps\": %d,\n \"eps0\": %.9g,\n \"seed\": %u,\n \"data\": \"%s\",\n \"chains\": [",
                 n_chains, stored_all, P, o.windows, o.chains, model.d0, model.d1, model.n, P,
                 model.lik_kind == BNNHMC_LIK_GAUSSIAN ? "gaussian" : "student_t", model.lik_scale,
                 model.lik_kind == BNNHMC_LIK_GAUSSIAN ? 0.0 : model.lik_df, model.prior_scale,
                 hmc.leapfrog_steps, hmc.burn_in, hmc.adapt_steps, (double)hmc.eps0, hmc.seed,
                 o.data.empty() ? "synthetic: features ~ N(0,1), teacher MLP ~ N(0, 0.1^2), noise sigma 0.01, "
                                  "key (seed, window)"
                                : o.data.c_str());
    for (int c = 0; c < n_chains; ++c) {
      float ceps = 0;
      int cacc = 0, cdone = 0;
      CHECK(bnnhmc_get_chain_state(s, c, nullptr, nullptr, &ceps, &cdone, &cacc));
      std::fprintf(mj, "%s\n  {\"chain\": %d, \"window\": %d, \"final_eps\": %.9g, \"transitions\": %d, "
                       "\"accepted\": %d}",
                   c ? "," : "", c, c / o.chains, (double)ceps, cdone, cacc);
    }
    std::fprintf(mj, "\n ]\n}\n");
    std::fclose(mj);
    std::printf("Wrote %d chain(s) x %d samples x %d floats to %s (metadata in %s)\n", n_chains, stored_all,
                P, o.dump.c_str(), meta.c_str());
  }
  double l1 = 0, l2 = 0, fl = 0;
  if (hmc.n_samples > 0) {
    CHECK(bnnhmc_final_loss(s, 0, &l1, &l2, &fl));
    std::printf("Final loss1: %g, loss2: %g, full loss: %g\n", l1, l2, fl);
  }
  if (o.chains > 1 && hmc.n_samples >= 8) {
    // convergence over the chains of window 0: worst split R-hat and smallest effective sample size
    std::vector<double> rhat(P), ess(P);
    CHECK(bnnhmc_window_diagnostics(s, 0, rhat.data(), ess.data()));
    double worst = 0, least = 1e300;
    for (int p = 0; p < P; ++p) {
      if (rhat[p] > worst) worst = rhat[p];
      if (ess[p] < least) least = ess[p];
    }
    std::printf("Window 0, %d chains: max split R-hat %.4f, min effective sample size %.1f of %d draws\n",
                o.chains, worst, least, o.chains * hmc.n_samples);
  }
  float eps = 0;
  int n_acc = 0, n_done = 0;
  CHECK(bnnhmc_get_chain_state(s, 0, nullptr, nullptr, &eps, &n_done, &n_acc));
  double kernel_ms = 0;
  long launches = 0, evals = 0;
  int wgs = 0;
  CHECK(bnnhmc_get_timing(s, &kernel_ms, &launches, &evals, &wgs));
  const double t_ms = std::chrono::duration<double, std::milli>(t_end - t_start).count();
  std::printf("Chain 0: %d/%d transitions accepted, final eps %g\n", n_acc, n_done, eps);
  std::printf("MCMC (%d burn in, %d sample steps, %d leap-frog steps) done in %.0fms; %ld gradient "
              "evaluations, %.1f evals/s (device %.0fms).\n",
              hmc.burn_in, hmc.n_samples, hmc.leapfrog_steps, t_ms, evals, evals / (t_ms * 1e-3),
              kernel_ms);
  int per_launch = 0, per_chain = 0;
  double trial[2] = {0.0, 0.0};
  CHECK(bnnhmc_get_batching(s, &per_launch, &per_chain, trial));
  std::printf("Launches of %d chain(s) on %d workgroups each", per_launch, per_chain);
  if (trial[0] > 0.0)
    std::printf(" (last timed pair: rows of a launch within 1.4 times the memory-side cache %.0f evals/s, as many chains "
                "as fit the device %.0f evals/s)", trial[0], trial[1]);
  std::printf(".\n");
  if (o.windows * o.chains == 1)
    std::printf("Expected time for 200 sequential passes: %.3fh. Good bye!\n", 200 * (t_ms / 3600000.0));
  CHECK(bnnhmc_destroy(s));
  return 0;
}
