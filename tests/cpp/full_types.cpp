// The full type configuration of the host layer (compile with -DEGEN_FULLTYPE
// and link libtenncor_host_full): what the reference generates from
// cfg/fulltype.yml:1-34 -- the enum in the key order of the file
// (tools/egen/plugins/dtypes.py:155-159), names, C types, precisions -- and
// what the node API does with it: leaves of every type, promotion of mixed
// operands to the most precise one through an inserted CAST
// (tenncor/eteq/make.hpp: make_funcattr), the CAST functor's `dtype`
// attribute.  Builds graphs only: no GPU is needed.
// Prints one line per failed expectation and exits with their count.
#ifndef EGEN_FULLTYPE
#error "compile with -DEGEN_FULLTYPE"
#endif
#include <cstdio>
#include <string>
#include <vector>

#include "eteq.hpp"

static int failures = 0;

#define EXPECT(COND) do { if (!(COND)) { ++failures; std::printf("%s:%d: expected %s\n", __FILE__, __LINE__, #COND); } } while (0)

template <typename T>
static teq::TensptrT var_of (const char* label, teq::Shape shape = teq::Shape({3, 2}))
{
	std::vector<T> data(shape.n_elems(), (T) 3);
	return eteq::make_variable<T>(data.data(), shape, label);
}

template <typename T>
static void check_leaf (egen::_GENERATED_DTYPE code, const char* name, size_t bytes)
{
	teq::TensptrT v = var_of<T>(name);
	EXPECT(v->get_meta().type_code() == (size_t) code);
	EXPECT(v->get_meta().type_label() == name);
	EXPECT(v->get_meta().type_size() == bytes);
	EXPECT(egen::get_type<T>() == code);
	EXPECT(egen::name_type(code) == name);
	EXPECT(egen::get_type(std::string(name)) == code);
	EXPECT(egen::type_size(code) == bytes);
	// a unary functor keeps the type of its operand
	teq::TensptrT f = eteq::make_functor(egen::SQUARE, {v});
	EXPECT(f->get_meta().type_code() == (size_t) code);
	// dispatch by code reaches the C type
	size_t seen = 0;
#define SIZE_OF(CT) seen = sizeof(CT);
	TYPE_LOOKUP(SIZE_OF, code)
#undef SIZE_OF
	EXPECT(seen == bytes);
}

static egen::_GENERATED_DTYPE type_of (const teq::TensptrT& tens)
{
	return (egen::_GENERATED_DTYPE) tens->get_meta().type_code();
}

int main (void)
{
	// cfg/fulltype.yml key order
	EXPECT(1 == egen::DOUBLE && 2 == egen::FLOAT && 3 == egen::INT8 && 4 == egen::UINT8 && 5 == egen::INT16);
	EXPECT(6 == egen::UINT16 && 7 == egen::INT32 && 8 == egen::UINT32 && 9 == egen::INT64 && 10 == egen::UINT64);
	EXPECT(11 == egen::_N_GENERATED_DTYPES && egen::FLOAT == egen::default_dtype);
	// cfg/fulltype.yml `precision`
	const egen::_GENERATED_DTYPE ascending[] = {egen::INT8, egen::UINT8, egen::INT16, egen::UINT16, egen::INT32,
		egen::UINT32, egen::INT64, egen::UINT64, egen::FLOAT, egen::DOUBLE};
	for (size_t i = 0; i < 10; ++i) { EXPECT(egen::type_precision(ascending[i]) == i + 1); }
	EXPECT(0 == egen::type_precision(egen::BAD_TYPE) && "BAD_TYPE" == egen::name_type(egen::BAD_TYPE));
	EXPECT(egen::BAD_TYPE == egen::get_type(std::string("HALF")));
	// the device library numbers the types its own way, the same in both configurations
	EXPECT(1 == egen::device_type(egen::DOUBLE) && 2 == egen::device_type(egen::FLOAT) && 3 == egen::device_type(egen::INT32));
	EXPECT(4 == egen::device_type<int8_t>() && 5 == egen::device_type<uint8_t>() && 6 == egen::device_type<int16_t>());
	EXPECT(7 == egen::device_type<uint16_t>() && 8 == egen::device_type<uint32_t>() && 9 == egen::device_type<int64_t>());
	EXPECT(10 == egen::device_type<uint64_t>() && 0 == egen::device_type(egen::BAD_TYPE));

	check_leaf<double>(egen::DOUBLE, "DOUBLE", 8);
	check_leaf<float>(egen::FLOAT, "FLOAT", 4);
	check_leaf<int8_t>(egen::INT8, "INT8", 1);
	check_leaf<uint8_t>(egen::UINT8, "UINT8", 1);
	check_leaf<int16_t>(egen::INT16, "INT16", 2);
	check_leaf<uint16_t>(egen::UINT16, "UINT16", 2);
	check_leaf<int32_t>(egen::INT32, "INT32", 4);
	check_leaf<uint32_t>(egen::UINT32, "UINT32", 4);
	check_leaf<int64_t>(egen::INT64, "INT64", 8);
	check_leaf<uint64_t>(egen::UINT64, "UINT64", 8);

	// mixed operands: the most precise type wins and the others are cast to it
	teq::TensptrT i8 = var_of<int8_t>("i8"), u16 = var_of<uint16_t>("u16"), i64 = var_of<int64_t>("i64");
	teq::TensptrT u64 = var_of<uint64_t>("u64"), f32 = var_of<float>("f32"), f64 = var_of<double>("f64");
	teq::TensptrT sum = eteq::make_functor(egen::ADD, {i8, u16});
	EXPECT(egen::UINT16 == type_of(sum));
	{
		auto f = dynamic_cast<teq::iFunctor*>(sum.get());
		EXPECT(nullptr != f);
		auto args = f->get_args();
		EXPECT(2 == args.size() && args[1] == u16);
		auto cast = dynamic_cast<teq::iFunctor*>(args[0].get());
		EXPECT(nullptr != cast && cast->get_opcode().code_ == (size_t) egen::CAST);
		EXPECT(nullptr != cast && egen::UINT16 == type_of(args[0]) && cast->get_args()[0] == i8);
	}
	EXPECT(egen::UINT64 == type_of(eteq::make_functor(egen::MUL, {i64, u64})));
	EXPECT(egen::FLOAT == type_of(eteq::make_functor(egen::SUB, {u64, f32})));
	EXPECT(egen::DOUBLE == type_of(eteq::make_functor(egen::MAX, {f32, i8, f64})));
	EXPECT(egen::INT64 == type_of(eteq::make_functor(egen::ADD, {i8, i64, u16})));

	// an explicit CAST names its target in the `dtype` attribute; onto its own type it is no node at all
	{
		marsh::Maps attrs;
		eigen::Packer<egen::_GENERATED_DTYPE>().pack(attrs, egen::UINT8);
		teq::TensptrT narrowed = eteq::make_funcattr(egen::CAST, {i64}, attrs);
		EXPECT(egen::UINT8 == type_of(narrowed));
		marsh::Maps same;
		eigen::Packer<egen::_GENERATED_DTYPE>().pack(same, egen::INT64);
		EXPECT(eteq::make_funcattr(egen::CAST, {i64}, same) == i64);
	}

	// type_convert reads every type
	{
		uint8_t bytes[3] = {0, 200, 255};
		double out[3];
		egen::type_convert<double>(out, bytes, egen::UINT8, 3);
		EXPECT(0 == out[0] && 200 == out[1] && 255 == out[2]);
		int64_t wide[2] = {-5, 70000};
		int16_t narrow[2];
		egen::type_convert<int16_t>(narrow, wide, egen::INT64, 2);
		EXPECT(-5 == narrow[0] && (int16_t) 70000 == narrow[1]);
	}
	std::printf("%d failure(s)\n", failures);
	return failures > 255 ? 255 : failures;
}
