// The reference's unit tests for the hot path (src/module/linear.rs:97-131, relu.rs:38-57,
// identity.rs:35-51, sequential.rs:119-172, optim/sgd.rs:34-43) written against the C++ mirror.
#include <cmath>
#include <cstdio>
#include <vector>

#include "rstorch.hpp"

using namespace rstorch;

static int failures = 0;
#define EXPECT(cond)                                                        \
  do {                                                                      \
    if (!(cond)) { std::printf("FAILED %s:%d  %s\n", __FILE__, __LINE__, #cond); ++failures; } \
  } while (0)

// assert_array_eq! of the reference (src/lib.rs:27-49): shape + absolute tolerance 1e-6
static bool array_eq(const Array2& a, const Array2& b, double tol = 1e-6) {
  if (!a.same_shape(b)) return false;
  auto x = a.to_host(), y = b.to_host();
  for (size_t i = 0; i < x.size(); ++i)
    if (!(std::fabs(x[i] - y[i]) <= tol)) return false;
  return true;
}

struct FixedInit : InitParameters {
  Array2 weight(size_t, size_t) const override { return Array2{{1.0, 0.5}}; }
  Array2 bias(size_t, size_t) const override { return Array2{{10.0}}; }
};

template <class F> static bool panics(F f) {
  try { f(); } catch (const Panic&) { return true; }
  return false;
}

int main() {
  try {
    {  // linear.rs:97-105
      Linear m = Linear::new_with_kernel(2, 1, FixedInit());
      Array2 out = m.forward(Array2{{1.0, 2.0}, {3.0, -4.0}, {-5.0, -6.0}});
      EXPECT(array_eq(out, Array2{{12.0}, {11.0}, {2.0}}));
    }
    {  // linear.rs:107-131
      Linear m = Linear::new_with_kernel(2, 1, FixedInit());
      m.forward(Array2{{1.0, 2.0}, {3.0, -4.0}, {-5.0, -6.0}, {-7.0, 8.0}});
      Array2 gx = m.backward(Array2::ones(4, 1));
      EXPECT(m.grad_weight().same_shape(m.weight()) && m.grad_bias().same_shape(m.bias()));
      EXPECT(array_eq(m.grad_weight(), Array2{{-2.0, 0.0}}));
      EXPECT(array_eq(m.grad_bias(), Array2{{1.0}}));
      EXPECT(array_eq(gx, Array2{{1.0, 0.5}, {1.0, 0.5}, {1.0, 0.5}, {1.0, 0.5}}));
      EXPECT(panics([&] { m.backward(Array2::ones(4, 1)); }));  // cache consumed (linear.rs:61)
    }
    {  // relu.rs:38-57
      ReLU m;
      EXPECT(array_eq(m.forward(Array2{{1.0, 2.0}, {3.0, -4.0}, {-5.0, -6.0}}),
                      Array2{{1.0, 2.0}, {3.0, 0.0}, {0.0, 0.0}}));
      EXPECT(array_eq(m.backward(Array2::ones(3, 2)), Array2{{1.0, 1.0}, {1.0, 0.0}, {0.0, 0.0}}));
      EXPECT(panics([&] { m.backward(Array2::ones(3, 2)); }));
    }
    {  // softmax.rs:85-113
      Softmax m;
      auto out = m.forward(Array2{{1.0, 10.0}, {-3.0, 4.0}, {5.0, 6.0}}).to_host();
      EXPECT(std::fabs(out[0] + out[1] - 1.0) < 1e-6 && out[0] + out[1] + out[2] + out[3] + out[4] + out[5] == 3.0);
      Softmax b;
      b.forward(Array2{{1.0, 2.0}, {3.0, 4.0}, {5.0, 6.0}});
      EXPECT(array_eq(b.backward(Array2::ones(3, 2)), Array2{{-0.41, -1.55}, {-0.41, -1.55}, {-0.41, -1.55}}, 0.01));
      auto col = Softmax::with_axis(0).forward(Array2{{1.0, 2.0}, {3.0, 4.0}, {5.0, 6.0}}).to_host();
      EXPECT(col[0] + col[1] + col[2] + col[3] + col[4] + col[5] == 2.0);
    }
    {  // identity.rs:35-51
      Identity m;
      Array2 d{{1.0, 2.0}, {3.0, 4.0}, {5.0, 6.0}};
      EXPECT(array_eq(m.forward(d), d) && array_eq(m.backward(d), d));
    }
    {  // sgd.rs:34-43
      SGD optim(0.1);
      Linear linear(2, 2);
      auto w0 = linear.weight().to_host();
      EXPECT(panics([&] { optim.step(linear); }));  // no gradient yet (linear.rs:72)
      linear.forward(Array2::zeros(2, 2));
      linear.backward(Array2::zeros(2, 2));
      optim.step(linear);
      EXPECT(linear.weight().to_host() == w0);
    }
    {  // sequential.rs:119-172 plus the container operations
      Sequential module = sequential(Linear(3, 10), ReLU(), Linear(10, 100), ReLU(), Linear(100, 2), Softmax());
      EXPECT(module.len() == 6 && !module.is_empty());
      Array2 out = module.forward(Array2{{1.0, 2.0, 3.0}, {-4.0, -5.0, -6.0}});
      EXPECT(out.nrows() == 2 && out.ncols() == 2);
      Array2 gin = module.backward(Array2{{1.0, 2.0}, {3.0, -4.0}});
      EXPECT(gin.nrows() == 2 && gin.ncols() == 3);
      EXPECT(module.parameters().size() == 6);
      EXPECT(module.remove(9) == nullptr);
      module.insert(0, Identity());
      module.push(ReLU());
      EXPECT(module.len() == 8);
      EXPECT(module.forward(Array2{{1.0, 2.0, 3.0}}).ncols() == 2);
    }
    {  // fused Sequential == layer-by-layer calls, bit for bit, and the loss/accuracy path
      Linear a(20, 30), b(30, 4);
      Linear a2 = a, b2 = b;  // shares the device weights (read-only here)
      Array2 x = Array2::normal(16, 20, 1, 1, 0.0, 1.0), y = Array2::one_hot(16, 4, 1, 2);
      ReLU r;
      Array2 manual = b.forward(r.forward(a.forward(x)));
      Sequential s;
      s.push(std::move(a2)); s.push(ReLU()); s.push(std::move(b2));
      Array2 fused = s.forward(x);
      EXPECT(manual.to_host() == fused.to_host());
      CrossEntropyLoss l1, l2;
      double v1 = l1.forward(manual.clone(), y.clone()), v2 = l2.forward(fused.clone(), y.clone());
      EXPECT(v1 == v2 && std::isfinite(v1));
      EXPECT(rstorch::utils::accuracy(manual, y) == rstorch::utils::accuracy(fused, y));
      Array2 g1 = a.backward(r.backward(b.backward(l1.backward())));
      Array2 g2 = s.backward(l2.backward());
      EXPECT(g1.to_host() == g2.to_host());
      EXPECT(panics([&] { l1.backward(); }));
      EXPECT(panics([&] { CrossEntropyLoss().forward(Array2::zeros(2, 3), Array2::zeros(2, 4)); }));
      Array2 bad = Array2::full(2, 3, std::nan(""));
      EXPECT(panics([&] { CrossEntropyLoss().forward(bad, Array2::zeros(2, 3)); }));
    }
    {  // the compiled Sequential (forward graph, backward deferred to the optimiser step) against the
       // same network run layer by layer: every observable value, bit for bit
      struct Given : InitParameters {
        Array2 w;
        explicit Given(Array2 a) : w(std::move(a)) {}
        Array2 weight(size_t, size_t) const override { return w.clone(); }
      };
      auto make = [&](bool compile) {
        Sequential m = sequential(Identity(), Linear::new_with_kernel(24, 40, Given(Array2::normal(40, 24, 9, 1, 0.0, 0.2))),
                                  ReLU(), Linear::new_with_kernel(40, 40, Given(Array2::normal(40, 40, 9, 2, 0.0, 0.15))),
                                  ReLU(), Linear::new_with_kernel(40, 6, Given(Array2::normal(6, 40, 9, 3, 0.0, 0.15))));
        m.set_compile(compile);
        return m;
      };
      Sequential fast = make(true), slow = make(false);
      CrossEntropyLoss lf, ls;
      SGD of(0.1), os(0.1);
      auto same_parameters = [&] {
        Parameters pf = fast.parameters(), ps = slow.parameters();
        bool ok = pf.size() == ps.size();
        for (size_t i = 0; ok && i < pf.size(); ++i)
          ok = pf.iter()[i].parm->to_host() == ps.iter()[i].parm->to_host() &&
               pf.iter()[i].grad->to_host() == ps.iter()[i].grad->to_host();
        return ok;
      };
      EXPECT(panics([&] { fast.backward(Array2::ones(4, 6)); }));
      EXPECT(panics([&] { fast.parameters(); }));
      // (from the second step on the compiled form takes the loop for a training loop and launches the
      // input gradients of the upper layers behind the loss, before the host has it: steps 5-7 make it
      // drop or overwrite them)
      for (int step = 0; step < 9; ++step) {
        Array2 x = Array2::normal(48, 24, 5, 10 + step % 2, 0.0, 1.0), y = Array2::one_hot(48, 6, 5, 20 + step % 2);
        Array2 pf = fast.forward(x), ps = slow.forward(x);
        EXPECT(pf.to_host() == ps.to_host());
        EXPECT(lf.forward(pf.clone(), y.clone()) == ls.forward(ps.clone(), y.clone()));
        if (step == 1) {         // the input gradient kept and read before the step
          Array2 gf = fast.backward(lf.backward()), gs = slow.backward(ls.backward());
          EXPECT(gf.to_host() == gs.to_host());
        } else if (step == 2) {  // kept, read after the step: computed with the weights of before
          Array2 gf = fast.backward(lf.backward()), gs = slow.backward(ls.backward());
          of.step(fast); os.step(slow);
          EXPECT(gf.to_host() == gs.to_host());
          EXPECT(same_parameters());
          continue;
        } else if (step == 5) {  // somebody looks at the loss gradient before it goes into backward
          Array2 gf = lf.backward(), gs = ls.backward();
          EXPECT(gf.to_host() == gs.to_host());
          fast.backward(gf); slow.backward(gs);
        } else if (step == 6) {  // another gradient than the loss's own goes into backward
          (void)lf.backward(); (void)ls.backward();
          Array2 other = Array2::normal(48, 6, 5, 40, 0.0, 1.0);
          fast.backward(other.clone()); slow.backward(other.clone());
        } else if (step == 8) {  // a parameter is rewritten between the loss and the backward pass
          for (Sequential* m : {&fast, &slow}) {
            Parameters ps = m->parameters();
            Array2& w = *ps.iter()[4].parm;  // the last Linear's weight: its input gradient must see the new one
            std::vector<double> h = w.to_host();
            for (double& v : h) v *= 0.5;
            check(rst_upload(w.engine(), w.data(), h.data(), h.size()));
          }
          fast.backward(lf.backward()); slow.backward(ls.backward());
        } else if (step == 7) {  // the loss is computed twice on the same logits; the second gradient is used
          EXPECT(lf.forward(pf.clone(), y.clone()) == ls.forward(ps.clone(), y.clone()));
          fast.backward(lf.backward()); slow.backward(ls.backward());
        } else {
          fast.backward(lf.backward()); slow.backward(ls.backward());
        }
        if (step == 3) EXPECT(same_parameters());  // gradients read between backward and step
        if (step == 4) EXPECT(panics([&] { fast.backward(Array2::ones(48, 6)); }));  // consumed
        of.step(fast); os.step(slow);
        EXPECT(same_parameters());
      }
      // the layer list changes: the compiled form is dropped, the weights stay with their layers
      fast.push(ReLU()); slow.push(ReLU());
      fast.insert(1, Identity()); slow.insert(1, Identity());
      Array2 x = Array2::normal(8, 24, 5, 30, 0.0, 1.0);
      EXPECT(fast.forward(x).to_host() == slow.forward(x).to_host());
      Array2 gf = fast.backward(Array2::ones(8, 6)), gs = slow.backward(Array2::ones(8, 6));
      EXPECT(gf.to_host() == gs.to_host());
      EXPECT(same_parameters());
      std::unique_ptr<Module> taken = fast.remove(2);  // the first Linear leaves with its trained weights
      std::unique_ptr<Module> taken_slow = slow.remove(2);
      EXPECT(static_cast<Linear*>(taken.get())->weight().to_host() == static_cast<Linear*>(taken_slow.get())->weight().to_host());
    }
  } catch (const Panic& p) {
    std::printf("unexpected panic: %s\n", p.what());
    return 2;
  }
  if (failures == 0) std::printf("all mirror tests passed\n");
  return failures == 0 ? 0 : 1;
}
