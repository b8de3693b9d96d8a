// GGUF container reader and model loader (host code; the only device calls are the uploads).
//
// The reference reads GGUF through ggml's gguf_init_from_file and turns every tensor into a graph
// variable (tools/gguf/GGUFImporter.cpp:644-678): plain types keep their dtype, block-quantised types
// keep their raw payload plus (format, [N, K]) (:457-502), metadata values are widened to
// u64 / i64 / f64 / bool / string (:339-437) and the LLaMA hyper-parameters are parsed from
// "<architecture>.*" keys with the defaults and checks of ParseLLaMAHyperparameters (:505-642).
// This file does the same without ggml: it parses the published container layout (magic "GGUF",
// version 2 or 3, little-endian; key/value table; tensor directory; data section aligned to
// general.alignment, default 32) from a read-only mapping of the file, reports what it finds with
// the reference's messages, and hands the raw payloads to the decoder runtime.
#include "common.hpp"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cctype>
#include <cstring>
#include <string>
#include <string_view>
#include <unordered_map>
#include <vector>

namespace litenn_hip
{
	namespace
	{
		const char* kReadAction = "GGUF import";
		const char* kLtnnAction = "LiteNN model import";

		// gguf metadata value types (published container layout)
		enum GgufType : uint32_t
		{
			kU8 = 0, kI8, kU16, kI16, kU32, kI32, kF32, kBool, kString, kArray, kU64, kI64, kF64,
		};

		// ggml tensor types this reader knows the size of (ids of the published ggml_type enum)
		struct TypeInfo
		{
			int ggml_type;
			const char* name;
			int block_elements;
			int block_bytes;
			int fmt;   // QuantizedBlockFormat the backend executes, or -1
			int dtype; // DataType of a plain tensor, or -1
		};
		const TypeInfo kTypes[] = {
			{ 0, "f32", 1, 4, -1, LITENN_F32 },    { 1, "f16", 1, 2, -1, LITENN_F16 },
			{ 2, "q4_0", 32, 18, LITENN_FMT_Q4_0, -1 }, { 3, "q4_1", 32, 20, LITENN_FMT_Q4_1, -1 },
			{ 6, "q5_0", 32, 22, LITENN_FMT_Q5_0, -1 }, { 7, "q5_1", 32, 24, LITENN_FMT_Q5_1, -1 },
			{ 8, "q8_0", 32, 34, LITENN_FMT_Q8_0, -1 }, { 9, "q8_1", 32, 36, -1, -1 },
			{ 10, "q2_K", 256, 84, LITENN_FMT_Q2_K, -1 }, { 11, "q3_K", 256, 110, LITENN_FMT_Q3_K, -1 },
			{ 12, "q4_K", 256, 144, LITENN_FMT_Q4_K, -1 }, { 13, "q5_K", 256, 176, LITENN_FMT_Q5_K, -1 },
			{ 14, "q6_K", 256, 210, LITENN_FMT_Q6_K, -1 }, { 15, "q8_K", 256, 292, -1, -1 },
			{ 24, "i8", 1, 1, -1, LITENN_I8 },      { 26, "i32", 1, 4, -1, LITENN_I32 },
			{ 27, "i64", 1, 8, -1, LITENN_I64 },    { 28, "f64", 1, 8, -1, LITENN_F64 },
			{ 30, "bf16", 1, 2, -1, LITENN_BF16 },
			// plain DataTypes without a ggml id (a LiteNN archive can hold them): -(DataType + 1)
			{ -(LITENN_BOOL + 1), "bool", 1, 1, -1, LITENN_BOOL },   { -(LITENN_F8E4M3 + 1), "f8e4m3", 1, 1, -1, LITENN_F8E4M3 },
			{ -(LITENN_F8E5M2 + 1), "f8e5m2", 1, 1, -1, LITENN_F8E5M2 }, { -(LITENN_U8 + 1), "u8", 1, 1, -1, LITENN_U8 },
		};
		const TypeInfo* find_type(int ggml_type)
		{
			for (const TypeInfo& t : kTypes)
			{
				if (t.ggml_type == ggml_type)
				{
					return &t;
				}
			}
			return nullptr;
		}

		struct Value
		{
			uint32_t type = 0;      // GgufType
			uint32_t elem_type = 0; // arrays
			uint64_t count = 0;     // arrays
			uint64_t u = 0;
			int64_t i = 0;
			double f = 0.0;
			bool b = false;
			std::string s;
		};

		struct TensorEntry
		{
			std::string name;
			int ggml_type = 0;
			std::vector<uint64_t> ne; // fastest dimension first, as stored
			uint64_t offset = 0;      // relative to the data section
			uint64_t bytes = 0;
		};
	} // namespace
} // namespace litenn_hip

using namespace litenn_hip;

struct litenn_gguf
{
	std::string path;
	const uint8_t* base = nullptr;
	size_t size = 0;
	uint32_t version = 0;
	std::vector<std::pair<std::string, Value>> metadata;
	std::unordered_map<std::string, size_t> metadata_index;
	std::vector<TensorEntry> tensors;
	std::unordered_map<std::string, size_t> tensor_index;
	uint64_t data_offset = 0;
};

namespace
{
	struct Cursor
	{
		const litenn_gguf* g;
		size_t pos = 0;
		bool ok = true;

		template <typename T>
		T read()
		{
			T v{};
			if (!ok || pos + sizeof(T) > g->size)
			{
				ok = false;
				return v;
			}
			std::memcpy(&v, g->base + pos, sizeof(T));
			pos += sizeof(T);
			return v;
		}
		std::string read_string()
		{
			const uint64_t n = read<uint64_t>();
			if (!ok || n > g->size - pos)
			{
				ok = false;
				return {};
			}
			std::string s(reinterpret_cast<const char*>(g->base + pos), static_cast<size_t>(n));
			pos += static_cast<size_t>(n);
			return s;
		}
		void skip(uint64_t n)
		{
			if (!ok || n > g->size - pos)
			{
				ok = false;
				return;
			}
			pos += static_cast<size_t>(n);
		}
	};

	size_t scalar_size(uint32_t type)
	{
		switch (type)
		{
		case kU8: case kI8: case kBool: return 1;
		case kU16: case kI16: return 2;
		case kU32: case kI32: case kF32: return 4;
		case kU64: case kI64: case kF64: return 8;
		default: return 0;
		}
	}

	bool read_scalar(Cursor& c, uint32_t type, Value& v)
	{
		v.type = type;
		switch (type)
		{
		case kU8: v.u = c.read<uint8_t>(); break;
		case kI8: v.i = c.read<int8_t>(); break;
		case kU16: v.u = c.read<uint16_t>(); break;
		case kI16: v.i = c.read<int16_t>(); break;
		case kU32: v.u = c.read<uint32_t>(); break;
		case kI32: v.i = c.read<int32_t>(); break;
		case kF32: v.f = static_cast<double>(c.read<float>()); break;
		case kBool: v.b = c.read<uint8_t>() != 0; break;
		case kString: v.s = c.read_string(); break;
		case kU64: v.u = c.read<uint64_t>(); break;
		case kI64: v.i = c.read<int64_t>(); break;
		case kF64: v.f = c.read<double>(); break;
		default: return false;
		}
		return c.ok;
	}

	bool is_unsigned(uint32_t t) { return t == kU8 || t == kU16 || t == kU32 || t == kU64; }
	bool is_signed(uint32_t t) { return t == kI8 || t == kI16 || t == kI32 || t == kI64; }
	bool is_float(uint32_t t) { return t == kF32 || t == kF64; }

	const Value* find_value(const litenn_gguf* g, const std::string& key)
	{
		const auto it = g->metadata_index.find(key);
		return it == g->metadata_index.end() ? nullptr : &g->metadata[it->second].second;
	}

	// ReadSizeValue / ReadDoubleValue / ReadStringValue / ReadBoolValue, tools/gguf/GGUFImporter.cpp:66-147
	int value_as_size(const std::string& key, const Value& v, uint64_t& out)
	{
		if (is_unsigned(v.type))
		{
			out = v.u;
			return 0;
		}
		if (is_signed(v.type))
		{
			if (v.i < 0)
			{
				return fail(kReadAction, "GGUF metadata key '" + key + "' must be non-negative");
			}
			out = static_cast<uint64_t>(v.i);
			return 0;
		}
		return fail(kReadAction, "GGUF metadata key '" + key + "' must be an integer");
	}
	int value_as_double(const std::string& key, const Value& v, double& out)
	{
		if (is_float(v.type))
		{
			out = v.f;
			return 0;
		}
		if (is_unsigned(v.type))
		{
			out = static_cast<double>(v.u);
			return 0;
		}
		if (is_signed(v.type))
		{
			out = static_cast<double>(v.i);
			return 0;
		}
		return fail(kReadAction, "GGUF metadata key '" + key + "' must be numeric");
	}

	// Byte size of every tensor from its type and shape, checked against the file.  All arithmetic on
	// sizes and offsets read from the file is done without wrapping: a product or sum that would not
	// fit is a tensor that cannot lie inside the file.  `alignment` (0: none) is what every tensor
	// offset must be a multiple of (ggml refuses a GGUF whose tensor data is not aligned).
	int finish_tensors(litenn_gguf* g, const char* what, uint64_t alignment)
	{
		const std::string kind = what;
		if (g->data_offset > g->size)
		{
			return fail(kReadAction, "Failed to open GGUF file '" + g->path + "'");
		}
		const uint64_t data_bytes = g->size - g->data_offset;
		for (TensorEntry& t : g->tensors)
		{
			const TypeInfo* ti = find_type(t.ggml_type);
			if (!ti)
			{
				return fail(kReadAction, "Unsupported ggml tensor type '" + std::to_string(t.ggml_type) + "' for tensor '" +
				                             t.name + "'");
			}
			// no tensor inside the file has more elements than the file has bytes times the elements a
			// block holds (a block takes at least one byte)
			const uint64_t element_limit = data_bytes * static_cast<uint64_t>(ti->block_elements) + 1;
			uint64_t elements = 1;
			for (uint64_t n : t.ne)
			{
				if (n == 0 || n > (uint64_t{ 1 } << 40))
				{
					return fail(kReadAction, kind + " tensor '" + t.name + "' has non-positive dimension " + std::to_string(n));
				}
				if (elements > element_limit / n)
				{
					return fail(kReadAction, "Failed to read the payload of " + kind + " tensor '" + t.name +
					                             "': its shape holds more elements than the file has room for");
				}
				elements *= n;
			}
			const uint64_t row = t.ne.empty() ? 1 : t.ne[0];
			if (row % static_cast<uint64_t>(ti->block_elements) != 0)
			{
				return fail(kReadAction, kind + " tensor '" + t.name + "' has an invalid serialized byte size");
			}
			t.bytes = elements / ti->block_elements * ti->block_bytes; // elements <= data_bytes * block + 1: no wrap
			if (t.offset > data_bytes || t.bytes > data_bytes - t.offset)
			{
				return fail(kReadAction, "Failed to read " + std::to_string(t.bytes) + " bytes for " + kind + " tensor '" +
				                             t.name + "'");
			}
			if (alignment != 0 && t.offset % alignment != 0)
			{
				return fail(kReadAction, kind + " tensor '" + t.name + "' has offset " + std::to_string(t.offset) +
				                             ", which is not a multiple of the alignment " + std::to_string(alignment));
			}
		}
		return 0;
	}

	int parse(litenn_gguf* g)
	{
		Cursor c{ g };
		const uint32_t magic = c.read<uint32_t>();
		g->version = c.read<uint32_t>();
		if (!c.ok || magic != 0x46554747u || (g->version != 2 && g->version != 3))
		{
			return fail(kReadAction, "Failed to open GGUF file '" + g->path + "'");
		}
		const uint64_t n_tensors = c.read<uint64_t>();
		const uint64_t n_kv = c.read<uint64_t>();
		if (!c.ok || n_tensors > g->size || n_kv > g->size)
		{
			return fail(kReadAction, "Failed to open GGUF file '" + g->path + "'");
		}
		for (uint64_t i = 0; i < n_kv; ++i)
		{
			std::string key = c.read_string();
			const uint32_t type = c.read<uint32_t>();
			Value v;
			if (!c.ok)
			{
				break;
			}
			if (type == kArray)
			{
				v.type = kArray;
				v.elem_type = c.read<uint32_t>();
				v.count = c.read<uint64_t>();
				if (v.elem_type == kString)
				{
					for (uint64_t e = 0; e < v.count && c.ok; ++e)
					{
						c.skip(c.read<uint64_t>());
					}
				}
				else
				{
					const size_t es = scalar_size(v.elem_type);
					if (es == 0)
					{
						return fail(kReadAction, "Unsupported GGUF metadata array type '" + std::to_string(v.elem_type) + "'");
					}
					if (v.count > g->size)
					{
						c.ok = false;
					}
					c.skip(v.count * es);
				}
			}
			else if (!read_scalar(c, type, v))
			{
				if (c.ok)
				{
					return fail(kReadAction, "Unsupported GGUF metadata type '" + std::to_string(type) + "'");
				}
			}
			g->metadata_index.emplace(key, g->metadata.size());
			g->metadata.emplace_back(std::move(key), std::move(v));
		}
		for (uint64_t i = 0; i < n_tensors && c.ok; ++i)
		{
			TensorEntry t;
			t.name = c.read_string();
			const uint32_t rank = c.read<uint32_t>();
			if (!c.ok || rank > 4)
			{
				c.ok = false;
				break;
			}
			for (uint32_t d = 0; d < rank; ++d)
			{
				t.ne.push_back(c.read<uint64_t>());
			}
			t.ggml_type = static_cast<int>(c.read<uint32_t>());
			t.offset = c.read<uint64_t>();
			g->tensor_index.emplace(t.name, g->tensors.size());
			g->tensors.push_back(std::move(t));
		}
		if (!c.ok)
		{
			return fail(kReadAction, "Failed to open GGUF file '" + g->path + "'");
		}
		uint64_t alignment = 32;
		if (const Value* a = find_value(g, "general.alignment"))
		{
			if (value_as_size("general.alignment", *a, alignment) != 0)
			{
				return 1;
			}
			if (alignment == 0 || (alignment & (alignment - 1)) != 0)
			{
				return fail(kReadAction, "Failed to open GGUF file '" + g->path + "'");
			}
		}
		g->data_offset = (c.pos + alignment - 1) / alignment * alignment;
		return finish_tensors(g, "GGUF", alignment);
	}

	// ---- LiteNN model archive (.ltnn) ---------------------------------------------------------
	// SaveModel writes, in this order (Serialization/ModelIO.h:1291-1341): magic "LTNNMDL\0", u32
	// version, u64 forward subgraph, u8 + u64 optional backward subgraph, input and output names,
	// u64 variable count, variable names, metadata entries, then per variable a tensor (u32 DataType,
	// u64 rank, u64 dims, raw bytes; :592-612) and an optional QuantizationParams record (:281-338);
	// activation slots, tape slots and the subgraphs follow.  Everything a weight loader needs comes
	// before the graph, so the reader stops after the variables: an archive of an imported GGUF model
	// (block-quantised variables keep their raw payload as UInt8 with the format and the expressed
	// shape in the record, GGUFImporter.cpp:478-491; the GGUF key/values are the metadata entries)
	// is exposed through the same handle and accessors as a .gguf file.
	const char kLtnnMagic[8] = { 'L', 'T', 'N', 'N', 'M', 'D', 'L', '\0' };

	size_t dtype_bytes(uint32_t dtype)
	{
		switch (dtype)
		{
		case LITENN_F32: case LITENN_I32: return 4;
		case LITENN_F64: case LITENN_I64: return 8;
		case LITENN_F16: case LITENN_BF16: return 2;
		case LITENN_BOOL: case LITENN_F8E4M3: case LITENN_F8E5M2: case LITENN_I8: case LITENN_U8: return 1;
		default: return 0;
		}
	}

	int dtype_to_type_id(uint32_t dtype)
	{
		switch (dtype)
		{
		case LITENN_F32: return 0;
		case LITENN_F16: return 1;
		case LITENN_I8: return 24;
		case LITENN_I32: return 26;
		case LITENN_I64: return 27;
		case LITENN_F64: return 28;
		case LITENN_BF16: return 30;
		default: return -(static_cast<int>(dtype) + 1);
		}
	}

	// QuantizedBlockFormat (Quantization.h:31-62) -> ggml type id, 0 when this reader has no size for it
	int block_format_to_type_id(uint32_t fmt)
	{
		static const int ids[] = { 0, 2, 3, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15 }; // Scalar, Q4_0 .. Q8_K
		return fmt < sizeof(ids) / sizeof(ids[0]) ? ids[fmt] : 0;
	}

	int parse_ltnn(litenn_gguf* g)
	{
		const auto bad = [&]() { return fail(kLtnnAction, "LiteNN model is truncated or unreadable"); };
		Cursor c{ g };
		c.skip(sizeof(kLtnnMagic));
		g->version = c.read<uint32_t>();
		if (!c.ok)
		{
			return bad();
		}
		// ModelIO.h:1361-1364; variable names and metadata exist from version 6 on (:1386-1390)
		if (g->version == 0 || g->version > 18)
		{
			return fail(kLtnnAction, "Unsupported LiteNN model version");
		}
		if (g->version < 6)
		{
			return fail(kLtnnAction, "LiteNN model version " + std::to_string(g->version) +
			                             " has no variable names; version 6 or later is needed");
		}
		c.read<uint64_t>(); // forward subgraph
		if (c.read<uint8_t>() != 0)
		{
			c.read<uint64_t>(); // backward subgraph
		}
		for (int list = 0; list < 2 && c.ok; ++list) // input names, output names
		{
			const uint64_t n = c.read<uint64_t>();
			for (uint64_t i = 0; i < n && c.ok; ++i)
			{
				c.skip(c.read<uint64_t>());
			}
		}
		const uint64_t n_vars = c.read<uint64_t>();
		const uint64_t n_names = c.read<uint64_t>();
		if (!c.ok || n_vars > g->size || n_names > g->size)
		{
			return bad();
		}
		std::vector<std::string> names;
		for (uint64_t i = 0; i < n_names && c.ok; ++i)
		{
			names.push_back(c.read_string());
		}
		if (c.ok && n_names != n_vars)
		{
			return fail(kLtnnAction, "LiteNN model names " + std::to_string(n_names) + " variables but holds " +
			                             std::to_string(n_vars));
		}
		// metadata entries (ModelIO.h:27-39,447-505)
		const uint64_t n_meta = c.read<uint64_t>();
		for (uint64_t i = 0; i < n_meta && c.ok; ++i)
		{
			std::string key = c.read_string();
			const uint32_t kind = c.read<uint32_t>();
			Value v;
			switch (kind)
			{
			case 0: v.type = kI64; v.i = c.read<int64_t>(); break;
			case 1: v.type = kU64; v.u = c.read<uint64_t>(); break;
			case 2: v.type = kF64; v.f = c.read<double>(); break;
			case 3:
			{
				const uint8_t b = c.read<uint8_t>();
				if (c.ok && b > 1)
				{
					return fail(kLtnnAction, "Invalid boolean value in LiteNN model metadata");
				}
				v.type = kBool;
				v.b = b != 0;
				break;
			}
			case 4: v.type = kString; v.s = c.read_string(); break;
			case 5: case 6: case 7: case 8:
			{
				static const uint32_t elem[] = { kI64, kU64, kF64, kBool };
				v.type = kArray;
				v.elem_type = elem[kind - 5];
				v.count = c.read<uint64_t>();
				if (v.count > g->size)
				{
					c.ok = false;
				}
				c.skip(v.count * (kind == 8 ? 1 : 8));
				break;
			}
			case 9:
				v.type = kArray;
				v.elem_type = kString;
				v.count = c.read<uint64_t>();
				for (uint64_t e = 0; e < v.count && c.ok; ++e)
				{
					c.skip(c.read<uint64_t>());
				}
				break;
			default:
				if (c.ok)
				{
					return fail(kLtnnAction, "LiteNN model contains an unknown metadata value kind");
				}
			}
			g->metadata_index.emplace(key, g->metadata.size());
			g->metadata.emplace_back(std::move(key), std::move(v));
		}
		for (uint64_t i = 0; i < n_vars && c.ok; ++i)
		{
			TensorEntry t;
			t.name = names[i];
			const uint32_t dtype = c.read<uint32_t>();
			const uint64_t rank = c.read<uint64_t>();
			if (!c.ok || rank > 16)
			{
				return bad();
			}
			std::vector<uint64_t> dims;
			uint64_t elements = 1;
			for (uint64_t d = 0; d < rank; ++d)
			{
				dims.push_back(c.read<uint64_t>());
				if (!c.ok || (dims.back() != 0 && elements > g->size / dims.back()))
				{
					return bad();
				}
				elements *= dims.back();
			}
			const size_t es = dtype_bytes(dtype);
			if (es == 0)
			{
				return fail(kLtnnAction, "LiteNN model variable '" + t.name + "' has an unknown data type");
			}
			const uint64_t payload = elements * es;
			t.offset = c.pos;
			c.skip(payload);
			const uint8_t has_q = c.read<uint8_t>();
			if (c.ok && has_q > 1)
			{
				return fail(kLtnnAction, "Invalid quantization metadata presence flag");
			}
			std::vector<uint64_t> shape = dims;
			t.ggml_type = dtype_to_type_id(dtype);
			if (has_q == 1)
			{
				const uint32_t scheme = c.read<uint32_t>();
				c.read<uint32_t>(); // granularity
				const uint32_t block_format = c.read<uint32_t>();
				c.read<uint32_t>(); // storage type
				c.read<uint32_t>(); // expressed type
				c.read<int64_t>();  // axis
				c.read<uint64_t>(); // group size
				const uint64_t n_scales = c.read<uint64_t>();
				c.skip(n_scales > g->size ? g->size + 1 : n_scales * 4);
				const uint64_t n_zero = c.read<uint64_t>();
				c.skip(n_zero > g->size ? g->size + 1 : n_zero * 4);
				const uint64_t n_expr = c.read<uint64_t>();
				if (!c.ok || n_expr > 16)
				{
					return bad();
				}
				std::vector<uint64_t> expressed;
				for (uint64_t d = 0; d < n_expr; ++d)
				{
					expressed.push_back(c.read<uint64_t>());
				}
				// QuantizationScheme::Block with a ggml format: the payload is raw blocks
				if (scheme == 1 && block_format != 0)
				{
					const int id = block_format_to_type_id(block_format);
					if (id == 0 || dtype != LITENN_U8)
					{
						return fail(kLtnnAction, "LiteNN model variable '" + t.name +
						                             "' uses a block format this reader has no layout for");
					}
					t.ggml_type = id;
					shape = expressed;
				}
			}
			if (shape.size() > 4)
			{
				return fail(kLtnnAction, "LiteNN model variable '" + t.name + "' has more than four dimensions");
			}
			t.ne.assign(shape.rbegin(), shape.rend()); // stored slowest dimension first
			t.bytes = payload;
			g->tensor_index.emplace(t.name, g->tensors.size());
			g->tensors.push_back(std::move(t));
		}
		if (!c.ok)
		{
			return bad();
		}
		g->data_offset = 0;
		// sizes implied by type and shape must be the payload sizes read above
		std::vector<uint64_t> payloads;
		for (const TensorEntry& t : g->tensors)
		{
			payloads.push_back(t.bytes);
		}
		if (finish_tensors(g, "LiteNN model", 0) != 0)
		{
			return 1;
		}
		for (size_t i = 0; i < g->tensors.size(); ++i)
		{
			if (g->tensors[i].bytes != payloads[i])
			{
				return fail(kLtnnAction, "LiteNN model variable '" + g->tensors[i].name +
				                             "' has an invalid serialized byte size");
			}
		}
		return 0;
	}

	void fill_info(const litenn_gguf* g, const TensorEntry& t, litenn_gguf_tensor* out)
	{
		const TypeInfo* ti = find_type(t.ggml_type);
		out->name = t.name.c_str();
		out->ggml_type = t.ggml_type;
		out->fmt = ti->fmt;
		out->dtype = ti->dtype;
		out->quantized = ti->block_elements > 1;
		out->rank = t.ne.size();
		for (size_t d = 0; d < 4; ++d)
		{
			// the reference reverses ggml's ne: slowest dimension first (TensorShape, GGUFImporter.cpp:206-221)
			out->shape[d] = d < t.ne.size() ? static_cast<size_t>(t.ne[t.ne.size() - 1 - d]) : 1;
		}
		out->file_offset = static_cast<size_t>(g->data_offset + t.offset);
		out->bytes = static_cast<size_t>(t.bytes);
		out->data = g->base + out->file_offset;
	}
} // namespace

extern "C" int litenn_gguf_open(const char* path, litenn_gguf** out)
{
	if (!path || !out)
	{
		return fail(kReadAction, "null argument");
	}
	*out = nullptr;
	const int fd = ::open(path, O_RDONLY);
	struct stat st{};
	if (fd < 0 || ::fstat(fd, &st) != 0 || st.st_size < 24)
	{
		if (fd >= 0)
		{
			::close(fd);
		}
		return fail(kReadAction, std::string("Failed to open GGUF file '") + path + "'");
	}
	void* map = ::mmap(nullptr, static_cast<size_t>(st.st_size), PROT_READ, MAP_PRIVATE, fd, 0);
	::close(fd);
	if (map == MAP_FAILED)
	{
		return fail(kReadAction, std::string("Failed to open GGUF payload stream '") + path + "'");
	}
	litenn_gguf* g = new litenn_gguf;
	g->path = path;
	g->base = static_cast<const uint8_t*>(map);
	g->size = static_cast<size_t>(st.st_size);
	const bool ltnn = std::memcmp(g->base, kLtnnMagic, sizeof(kLtnnMagic)) == 0;
	if ((ltnn ? parse_ltnn(g) : parse(g)) != 0)
	{
		litenn_gguf_close(g);
		return 1;
	}
	*out = g;
	return 0;
}

extern "C" void litenn_gguf_close(litenn_gguf* g)
{
	if (!g)
	{
		return;
	}
	if (g->base)
	{
		::munmap(const_cast<uint8_t*>(g->base), g->size);
	}
	delete g;
}

extern "C" size_t litenn_gguf_tensor_count(const litenn_gguf* g) { return g ? g->tensors.size() : 0; }
extern "C" size_t litenn_gguf_metadata_count(const litenn_gguf* g) { return g ? g->metadata.size() : 0; }
extern "C" unsigned litenn_gguf_version(const litenn_gguf* g) { return g ? g->version : 0; }

extern "C" int litenn_gguf_tensor_info(const litenn_gguf* g, size_t index, litenn_gguf_tensor* out)
{
	if (!g || !out || index >= g->tensors.size())
	{
		return fail(kReadAction, "tensor index out of range");
	}
	fill_info(g, g->tensors[index], out);
	return 0;
}

extern "C" int litenn_gguf_find_tensor(const litenn_gguf* g, const char* name, litenn_gguf_tensor* out)
{
	if (!g || !name || !out)
	{
		return fail(kReadAction, "null argument");
	}
	const auto it = g->tensor_index.find(name);
	if (it == g->tensor_index.end())
	{
		return fail(kReadAction, std::string("Missing GGUF tensor '") + name + "'");
	}
	fill_info(g, g->tensors[it->second], out);
	return 0;
}

extern "C" const char* litenn_gguf_metadata_key(const litenn_gguf* g, size_t index)
{
	return g && index < g->metadata.size() ? g->metadata[index].first.c_str() : nullptr;
}

static const Value* require(const litenn_gguf* g, const char* key)
{
	const Value* v = g && key ? find_value(g, key) : nullptr;
	if (!v)
	{
		fail(kReadAction, std::string("Missing GGUF metadata key '") + (key ? key : "") + "'");
	}
	return v;
}

extern "C" int litenn_gguf_metadata_u64(const litenn_gguf* g, const char* key, uint64_t* out)
{
	const Value* v = require(g, key);
	return v ? value_as_size(key, *v, *out) : 1;
}

extern "C" int litenn_gguf_metadata_f64(const litenn_gguf* g, const char* key, double* out)
{
	const Value* v = require(g, key);
	return v ? value_as_double(key, *v, *out) : 1;
}

extern "C" int litenn_gguf_metadata_str(const litenn_gguf* g, const char* key, const char** out)
{
	const Value* v = require(g, key);
	if (!v)
	{
		return 1;
	}
	if (v->type != kString)
	{
		return fail(kReadAction, std::string("GGUF metadata key '") + key + "' must be a string");
	}
	*out = v->s.c_str();
	return 0;
}

extern "C" int litenn_gguf_metadata_bool(const litenn_gguf* g, const char* key, int* out)
{
	const Value* v = require(g, key);
	if (!v)
	{
		return 1;
	}
	if (v->type != kBool)
	{
		return fail(kReadAction, std::string("GGUF metadata key '") + key + "' must be a bool");
	}
	*out = v->b ? 1 : 0;
	return 0;
}

extern "C" int litenn_gguf_metadata_array(const litenn_gguf* g, const char* key, unsigned* elem_type, size_t* count)
{
	const Value* v = require(g, key);
	if (!v)
	{
		return 1;
	}
	if (v->type != kArray)
	{
		return fail(kReadAction, std::string("GGUF metadata key '") + key + "' must be an array");
	}
	*elem_type = v->elem_type;
	*count = static_cast<size_t>(v->count);
	return 0;
}

// ParseLLaMAHyperparameters, tools/gguf/GGUFImporter.cpp:505-642, plus the vocabulary size the
// builder takes from token_embd.weight (tools/gguf/LLaMABuilder.cpp:685-703) and its refusal of
// rope scaling types it does not execute (:300-308).
extern "C" int litenn_gguf_llama_params(const litenn_gguf* g, litenn_hip_llama_params* out)
{
	if (!g || !out)
	{
		return fail(kReadAction, "null argument");
	}
	const char* arch_c = nullptr;
	if (litenn_gguf_metadata_str(g, "general.architecture", &arch_c) != 0)
	{
		return 1;
	}
	const std::string arch = arch_c;
	if (arch.empty())
	{
		return fail(kReadAction, "GGUF metadata key 'general.architecture' must not be empty");
	}
	const auto key = [&arch](const char* suffix) { return arch + "." + suffix; };
	uint64_t ctx = 0, emb = 0, blocks = 0, ff = 0, heads = 0, kv_heads = 0, rope_dims = 0;
	double eps = 0.0, base = 10000.0, scale = 1.0;
	if (litenn_gguf_metadata_u64(g, key("context_length").c_str(), &ctx) != 0 ||
	    litenn_gguf_metadata_u64(g, key("embedding_length").c_str(), &emb) != 0 ||
	    litenn_gguf_metadata_u64(g, key("block_count").c_str(), &blocks) != 0 ||
	    litenn_gguf_metadata_u64(g, key("feed_forward_length").c_str(), &ff) != 0 ||
	    litenn_gguf_metadata_u64(g, key("attention.head_count").c_str(), &heads) != 0 ||
	    litenn_gguf_metadata_f64(g, key("attention.layer_norm_rms_epsilon").c_str(), &eps) != 0)
	{
		return 1;
	}
	kv_heads = heads;
	if (find_value(g, key("attention.head_count_kv")) &&
	    litenn_gguf_metadata_u64(g, key("attention.head_count_kv").c_str(), &kv_heads) != 0)
	{
		return 1;
	}
	if (find_value(g, key("rope.freq_base")) && litenn_gguf_metadata_f64(g, key("rope.freq_base").c_str(), &base) != 0)
	{
		return 1;
	}
	if (find_value(g, key("rope.freq_scale")) && litenn_gguf_metadata_f64(g, key("rope.freq_scale").c_str(), &scale) != 0)
	{
		return 1;
	}
	if (find_value(g, key("rope.dimension_count")) &&
	    litenn_gguf_metadata_u64(g, key("rope.dimension_count").c_str(), &rope_dims) != 0)
	{
		return 1;
	}
	std::string scaling = "none";
	if (find_value(g, key("rope.scaling.type")))
	{
		const char* s = nullptr;
		if (litenn_gguf_metadata_str(g, key("rope.scaling.type").c_str(), &s) != 0)
		{
			return 1;
		}
		scaling = s;
		std::transform(scaling.begin(), scaling.end(), scaling.begin(),
		               [](unsigned char ch) { return static_cast<char>(std::tolower(ch)); });
	}
	if (find_value(g, key("rope.scaling.factor")))
	{
		double factor = 0.0;
		if (litenn_gguf_metadata_f64(g, key("rope.scaling.factor").c_str(), &factor) != 0)
		{
			return 1;
		}
		if (factor < 0.0)
		{
			return fail(kReadAction, "LLaMA rope.scaling.factor must be non-negative");
		}
		scale = factor == 0.0 ? 1.0 : 1.0 / factor;
	}
	if (ctx == 0 || emb == 0 || blocks == 0 || ff == 0)
	{
		return fail(kReadAction, "LLaMA hyperparameters must be greater than zero");
	}
	if (!(eps > 0.0))
	{
		return fail(kReadAction, "LLaMA attention.layer_norm_rms_epsilon must be greater than zero");
	}
	if (!(base > 0.0))
	{
		return fail(kReadAction, "LLaMA rope.freq_base must be greater than zero");
	}
	if (!(scale > 0.0))
	{
		return fail(kReadAction, "LLaMA rope.freq_scale must be greater than zero");
	}
	if (scaling != "none" && scaling != "linear" && scaling != "yarn" && scaling != "longrope")
	{
		return fail(kReadAction, "Unsupported LLaMA rope.scaling.type '" + scaling + "'");
	}
	if (heads == 0)
	{
		return fail(kReadAction, "LLaMA attention.head_count must be greater than zero");
	}
	if (emb % heads != 0)
	{
		return fail(kReadAction, "LLaMA embedding_length " + std::to_string(emb) +
		                             " must be divisible by attention.head_count " + std::to_string(heads));
	}
	const uint64_t head_dim = emb / heads;
	if (rope_dims == 0)
	{
		rope_dims = head_dim;
	}
	if (rope_dims > head_dim || rope_dims % 2 != 0)
	{
		return fail(kReadAction, "LLaMA rope.dimension_count must be an even value in [2, headDim]");
	}
	if (kv_heads == 0)
	{
		return fail(kReadAction, "LLaMA attention.head_count_kv must be greater than zero");
	}
	if (heads % kv_heads != 0)
	{
		return fail(kReadAction, "LLaMA attention.head_count " + std::to_string(heads) +
		                             " must be divisible by attention.head_count_kv " + std::to_string(kv_heads));
	}
	if (scaling == "yarn" || scaling == "longrope")
	{
		return fail(kReadAction, "Current LLaMA decode lowering preserves rope.scaling.* metadata but only executes "
		                         "none/linear scaling, got '" + scaling + "'");
	}
	litenn_gguf_tensor embd;
	if (litenn_gguf_find_tensor(g, "token_embd.weight", &embd) != 0)
	{
		return 1;
	}
	if (embd.rank != 2)
	{
		return fail(kReadAction, "GGUF tensor 'token_embd.weight' must be 2D for current LLaMA lowering");
	}
	if (embd.shape[1] != emb)
	{
		return fail(kReadAction, "GGUF tensor 'token_embd.weight' must have LiteNN shape [vocab, " + std::to_string(emb) +
		                             "] for the HIP decoder");
	}
	const uint64_t limit = 0x7fffffffu;
	if (ctx > limit || emb > limit || blocks > limit || ff > limit || embd.shape[0] > limit)
	{
		return fail(kReadAction, "LLaMA hyperparameters exceed 2^31-1");
	}
	out->block_count = static_cast<int32_t>(blocks);
	out->embedding_length = static_cast<int32_t>(emb);
	out->head_count = static_cast<int32_t>(heads);
	out->head_count_kv = static_cast<int32_t>(kv_heads);
	out->feed_forward_length = static_cast<int32_t>(ff);
	out->vocab_size = static_cast<int32_t>(embd.shape[0]);
	out->context_length = static_cast<int32_t>(ctx);
	out->rope_dimension_count = static_cast<int32_t>(rope_dims);
	out->rms_norm_epsilon = eps;
	out->rope_freq_base = base;
	out->rope_freq_scale = scale;
	return 0;
}

// ---- loader: GGUF file -> resident decoder -----------------------------------------------------

namespace litenn_hip
{
	int llama_adopt(litenn_hip_llama* model, void* device_ptr); // llama.hip: frees it with the model
}

namespace
{
	int upload(int dev, const litenn_gguf_tensor& t, void** out)
	{
		DeviceGuard guard(dev);
		if (!guard.ok())
		{
			return 1;
		}
		LITENN_HIP_TRY("GGUF upload", hipMalloc(out, t.bytes));
		const hipError_t e = hipMemcpy(*out, t.data, t.bytes, hipMemcpyHostToDevice);
		if (e != hipSuccess)
		{
			(void)hipFree(*out);
			*out = nullptr;
			return fail_hip("GGUF upload", e);
		}
		return 0;
	}

	// one tensor of the decoder: present in the file, 2-D [n, k] of an executable format (or 1-D f32
	// for the norm weights), uploaded and handed to the runtime
	int place(int dev, const litenn_gguf* g, litenn_hip_llama* model, const std::string& name, int which, int layer,
	          bool norm, bool optional)
	{
		litenn_gguf_tensor t;
		if (g->tensor_index.find(name) == g->tensor_index.end())
		{
			return optional ? 0 : fail(kReadAction, "Missing GGUF tensor '" + name + "'");
		}
		if (litenn_gguf_find_tensor(g, name.c_str(), &t) != 0)
		{
			return 1;
		}
		int fmt;
		size_t n, k;
		if (norm)
		{
			if (t.dtype != LITENN_F32 || t.rank != 1)
			{
				return fail(kReadAction, "GGUF tensor '" + name + "' must be a 1-D Float32 vector");
			}
			fmt = LITENN_FMT_F32;
			n = 1;
			k = t.shape[0];
		}
		else
		{
			if (t.rank != 2)
			{
				return fail(kReadAction, "GGUF tensor '" + name + "' must be 2D for current LLaMA lowering");
			}
			fmt = t.fmt >= 0 ? t.fmt : (t.dtype == LITENN_F32 ? LITENN_FMT_F32 : (t.dtype == LITENN_F16 ? LITENN_FMT_F16 : -1));
			if (fmt < 0)
			{
				return fail(kReadAction, "Unsupported ggml tensor type '" + std::string(find_type(t.ggml_type)->name) +
				                             "' for tensor '" + name + "'");
			}
			n = t.shape[0];
			k = t.shape[1];
		}
		void* dptr = nullptr;
		if (upload(dev, t, &dptr) != 0)
		{
			return 1;
		}
		if (litenn_hip::llama_adopt(model, dptr) != 0)
		{
			(void)hipFree(dptr);
			return 1;
		}
		return litenn_hip_llama_set_tensor(model, which, layer, fmt, dptr, n, k);
	}
} // namespace

extern "C" int litenn_hip_llama_load_gguf(int dev, const char* path, int kv_dtype, int32_t context_length,
                                          litenn_hip_llama** out)
{
	if (!out)
	{
		return fail(kReadAction, "null argument");
	}
	*out = nullptr;
	litenn_gguf* g = nullptr;
	if (litenn_gguf_open(path, &g) != 0)
	{
		return 1;
	}
	litenn_hip_llama_params p{};
	if (litenn_gguf_llama_params(g, &p) != 0)
	{
		litenn_gguf_close(g);
		return 1;
	}
	p.kv_dtype = kv_dtype;
	if (context_length > 0)
	{
		p.context_length = context_length;
	}
	litenn_hip_llama* model = nullptr;
	if (litenn_hip_llama_create(dev, &p, &model) != 0)
	{
		litenn_gguf_close(g);
		return 1;
	}
	int rc = place(dev, g, model, "token_embd.weight", LITENN_T_TOKEN_EMBD, -1, false, false);
	rc = rc ? rc : place(dev, g, model, "output_norm.weight", LITENN_T_OUTPUT_NORM, -1, true, false);
	// absent output.weight: the head is tied to the embedding (tools/gguf/LLaMABuilder.cpp:719-733)
	rc = rc ? rc : place(dev, g, model, "output.weight", LITENN_T_OUTPUT, -1, false, true);
	static const struct { const char* suffix; int which; bool norm; } kBlock[] = {
		{ "attn_norm.weight", LITENN_T_ATTN_NORM, true },    { "attn_q.weight", LITENN_T_ATTN_Q, false },
		{ "attn_k.weight", LITENN_T_ATTN_K, false },         { "attn_v.weight", LITENN_T_ATTN_V, false },
		{ "attn_output.weight", LITENN_T_ATTN_OUTPUT, false }, { "ffn_norm.weight", LITENN_T_FFN_NORM, true },
		{ "ffn_gate.weight", LITENN_T_FFN_GATE, false },     { "ffn_up.weight", LITENN_T_FFN_UP, false },
		{ "ffn_down.weight", LITENN_T_FFN_DOWN, false },
	};
	for (int layer = 0; layer < p.block_count && rc == 0; ++layer)
	{
		for (const auto& b : kBlock)
		{
			rc = place(dev, g, model, "blk." + std::to_string(layer) + "." + b.suffix, b.which, layer, b.norm, false);
			if (rc != 0)
			{
				break;
			}
		}
	}
	litenn_gguf_close(g);
	if (rc != 0)
	{
		const std::string keep = litenn_hip_last_error(); // llama_free must not hide the cause
		litenn_hip_llama_free(model);
		set_error(keep);
		return 1;
	}
	*out = model;
	return 0;
}
