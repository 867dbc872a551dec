// The sigmoid MLP of the reference's equation test (tenncor/test/
// test_equation.cpp:482-706, exactly the shapes of a two-layer dense network on
// a batch of three) built and evaluated from C++ through the host layer the way
// a tenncor checkout would: eteq::make_variable / make_functor, tcr::derive,
// teq::Evaluator on an eigen::Device, results read through device().data().
// Input: lines "name count v0 v1 ..." on stdin (in, w0, b0, w1, b1, out);
// output: the four gradients in the same format.  Needs a GPU.
#include <cstdio>
#include <iostream>
#include <map>
#include <string>
#include <vector>

#include "eteq.hpp"
#include "replay_eval.hpp"

// mlp_gradients [replay]: with "replay" the process-wide evaluator slot holds
// the recording evaluator (teq::set_eval) and the targets are evaluated four
// times with the input re-assigned in between: walk, record, replay, replay
int main (int argc, char** argv)
{
	const bool replay = argc > 1 && std::string(argv[1]) == "replay";
	std::map<std::string,std::vector<double>> in;
	std::string name;
	size_t n;
	while (std::cin >> name >> n)
	{
		std::vector<double> vals(n);
		for (double& v : vals) { std::cin >> v; }
		in.emplace(name, vals);
	}
	try
	{
		auto leaf = [&](const char* key, teq::Shape shape) -> teq::TensptrT
		{
			auto& vals = in.at(key);
			if (vals.size() != shape.n_elems()) { global::fatalf("%s: %d values", key, (int) vals.size()); }
			return eteq::make_variable<double>(vals.data(), shape, key);
		};
		teq::TensptrT x = leaf("in", teq::Shape({10, 3}));
		teq::TensptrT w0 = leaf("w0", teq::Shape({9, 10})), b0 = leaf("b0", teq::Shape({9}));
		teq::TensptrT w1 = leaf("w1", teq::Shape({5, 9})), b1 = leaf("b1", teq::Shape({5}));
		teq::TensptrT out = leaf("out", teq::Shape({5, 3}));

		auto layer = [](teq::TensptrT input, teq::TensptrT weight, teq::TensptrT bias)
		{
			auto product = eteq::make_functor(egen::MATMUL, {input, weight});
			auto biased = eteq::make_functor(egen::ADD, {product,
				eteq::make_functor(egen::EXTEND, {bias}, teq::DimsT{1, 3})});
			return eteq::make_functor(egen::SIGMOID, {biased});
		};
		auto sig1 = layer(layer(x, w0, b0), w1, b1);
		auto diff = eteq::make_functor(egen::SUB, {out, sig1});
		auto err = eteq::make_functor(egen::POW, {diff, eteq::make_constant_like<double>(2., diff)});

		teq::TensptrsT grads = tcr::derive(err, {w0, b0, w1, b1});
		eigen::Device device;
		teq::TensSetT targets;
		for (auto& g : grads) { targets.emplace(g.get()); }
		if (replay)
		{
			teq::set_eval(new eigen::ReplayEvaluator());
			auto input = std::static_pointer_cast<eteq::Variable<double>>(x);
			for (int pass = 0; pass < 4; ++pass)
			{
				input->assign(in.at("in").data(), input->shape()); // a new version: everything recomputes
				teq::get_eval().evaluate(device, targets, {});
			}
			auto stats = static_cast<eigen::ReplayEvaluator&>(teq::get_eval()).stats();
			std::printf("replayed %zu\n", (size_t) stats.replayed);
		}
		else
		{
			teq::Evaluator().evaluate(device, targets);
			teq::Evaluator().evaluate(device, targets); // nothing to do the second time
		}

		const char* names[] = {"gw0", "gb0", "gw1", "gb1"};
		for (size_t i = 0; i < grads.size(); ++i)
		{
			const double* data = (const double*) grads[i]->device().data();
			if (nullptr == data) { global::fatalf("%s holds no value", names[i]); }
			size_t count = grads[i]->shape().n_elems();
			std::printf("%s %zu", names[i], count);
			for (size_t j = 0; j < count; ++j) { std::printf(" %.17g", data[j]); }
			std::printf("\n");
		}
	}
	catch (std::exception& e)
	{
		std::printf("error %s\n", e.what());
		return 1;
	}
	return 0;
}
