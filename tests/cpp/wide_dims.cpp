// The build variant with dimensions wider than 16 bits (SDIM_BYTES,
// internal/teq/shape.hpp:27-33): the host layer compiled with -DSDIM_BYTES=4
// holds a dimension of 70000 where the default build's uint16_t could not.
// Builds graphs only: no GPU is needed.  Exits with the number of failures.
#include <cstdio>
#include <vector>

#include "eteq.hpp"

static_assert(sizeof(teq::DimT) == 4, "built without -DSDIM_BYTES=4");

static int failures = 0;

#define EXPECT(COND) do { if (!(COND)) { ++failures; std::printf("%s:%d: expected %s\n", __FILE__, __LINE__, #COND); } } while (0)

int main (void)
{
	teq::Shape wide({70000, 3});
	EXPECT(70000 == wide.at(0));
	EXPECT(3 == wide.at(1));
	EXPECT(210000 == wide.n_elems());
	EXPECT("[70000\\3\\1\\1\\1\\1\\1\\1]" == wide.to_string());

	std::vector<float> data(wide.n_elems(), 1.0f);
	teq::TensptrT leaf = eteq::make_variable<float>(data.data(), wide, "leaf");
	teq::TensptrT neg = eteq::make_functor(egen::NEG, {leaf});
	teq::TensptrT sum = eteq::make_functor(egen::ADD, {neg, leaf});
	teq::Shape got = sum->shape();
	EXPECT(70000 == got.at(0));
	EXPECT(210000 == got.n_elems());
	std::printf("%d failure(s)\n", failures);
	return failures;
}
