"""
TEST ORACLE - not part of the product.  Only tests, the smoke check and the benchmark's CPU-baseline leg may use it.

Emits, for one serialised expression DAG, the C++ text that the reference's code generator would emit for the same
DAG: one statement per registered expression, in registration order, with the reference's statement forms, inside
the reference's per-thread worker loop.  The results of the compiled code depend only on this sequence of typed C
operations and libm calls, so this restates "the reference's generated g++ C++ path".

Followed reference code (all in opveclib/expression.py):
  worker loop and function prologue ............ 569-593
  naming of expressions (e<N>, (*in<i>), ...) .. 320-333
  argument list (pointer to fixed-size array) .. 548-552, 1039-1045, 1111-1117
  POSITION ..................................... 1293-1306
  VARIABLE / CAST .............................. 1351-1352, 1386-1387
  ASSIGN_VARIABLE .............................. 1422-1423
  unary math table ............................. 1430-1456, 1479-1481
  limits ....................................... 1568-1572, 1587
  binary math table ............................ 1632-1672, 1739-1742
  local tensors ................................ 1788-1795
  ASSIGN_TENSOR / READ_TENSOR .................. 1881-1882, 1904-1905
  RANGE / ENDRANGE ............................. 1996-2006, 2021-2022
  IF / ELSEIF / ELSE / ENDIF ................... 2064-2065, 2115-2116, 2160-2161, 2182-2183
  generic wrapper: count and length checks, block split ... 611-673

Deviation (boundary only): the reference's wrapper receives std::vector<std::shared_ptr<InputParameter>> by value
(expression.py:657-660); this wrapper receives plain C arrays of ``ovl_tensor`` so that it can be driven without the
reference's header.  The checks it performs and the block split it computes are the same.

Pinned by tests/test_oracle_golden.py: README shift example, reference doctest tables for cumsum/cumprod, expm1 and
log1p edge vectors, clip / arange / dot-product / limits tests of the reference, numpy closed forms for every unary
and binary function, C truncation semantics for integer division and modulo.
"""

from opveclib_amd import language as lang

CTYPE = {
    lang.FLOAT32: 'float', lang.FLOAT64: 'double',
    lang.INT8: 'int8_t', lang.INT16: 'int16_t', lang.INT32: 'int32_t', lang.INT64: 'int64_tf',
    lang.UINT8: 'uint8_t', lang.UINT16: 'uint16_t', lang.UINT32: 'uint32_t', lang.UINT64: 'uint64_t'}

UNARY = {
    lang.ACOS: {lang.FLOAT32: 'acosf', lang.FLOAT64: 'acos'},
    lang.ASIN: {lang.FLOAT32: 'asinf', lang.FLOAT64: 'asin'},
    lang.ATAN: {lang.FLOAT32: 'atanf', lang.FLOAT64: 'atan'},
    lang.COS: {lang.FLOAT32: 'cosf', lang.FLOAT64: 'cos'},
    lang.COSH: {lang.FLOAT32: 'coshf', lang.FLOAT64: 'cosh'},
    lang.SIN: {lang.FLOAT32: 'sinf', lang.FLOAT64: 'sin'},
    lang.SINH: {lang.FLOAT32: 'sinhf', lang.FLOAT64: 'sinh'},
    lang.TAN: {lang.FLOAT32: 'tanf', lang.FLOAT64: 'tan'},
    lang.TANH: {lang.FLOAT32: 'tanhf', lang.FLOAT64: 'tanh'},
    lang.EXP: {lang.FLOAT32: 'expf', lang.FLOAT64: 'exp'},
    lang.LOG: {lang.FLOAT32: 'logf', lang.FLOAT64: 'log'},
    lang.LOG10: {lang.FLOAT32: 'log10f', lang.FLOAT64: 'log10'},
    lang.SQRT: {lang.FLOAT32: 'sqrtf', lang.FLOAT64: 'sqrt'},
    lang.CEIL: {lang.FLOAT32: 'ceilf', lang.FLOAT64: 'ceil'},
    lang.FLOOR: {lang.FLOAT32: 'floorf', lang.FLOAT64: 'floor'},
    lang.ABS: {lang.FLOAT32: 'fabsf', lang.FLOAT64: 'fabs', lang.INT8: 'abs_8', lang.INT16: 'abs_16',
               lang.INT32: 'abs', lang.INT64: 'labs'},
    lang.ISINF: {lang.FLOAT32: 'isinf', lang.FLOAT64: 'isinf'},
    lang.ISFINITE: {lang.FLOAT32: 'isfinite', lang.FLOAT64: 'isfinite'},
    lang.ISNAN: {lang.FLOAT32: 'isnan', lang.FLOAT64: 'isnan'},
}
_SIGNED_OR_FLOAT = (lang.FLOAT32, lang.FLOAT64, lang.INT8, lang.INT16, lang.INT32, lang.INT64)
UNARY[lang.NEGATE] = dict((t, '-') for t in _SIGNED_OR_FLOAT)
UNARY[lang.NOT] = dict((t, '!') for t in CTYPE)

INFIX = {lang.ADD: '+', lang.SUBTRACT: '-', lang.MULTIPLY: '*', lang.DIVIDE: '/', lang.MODULO: '%',
         lang.EQUAL: '==', lang.NOTEQUAL: '!=', lang.LESS: '<', lang.LESS_EQ: '<=', lang.GREATER: '>',
         lang.GREATER_EQ: '>=', lang.AND: '&&', lang.OR: '||'}

LIMITS = {lang.MIN_VALUE: {lang.FLOAT32: 'FLT_MIN', lang.FLOAT64: 'DBL_MIN'},
          lang.MAX_VALUE: {lang.FLOAT32: 'FLT_MAX', lang.FLOAT64: 'DBL_MAX'},
          lang.EPSILON: {lang.FLOAT32: 'FLT_EPSILON', lang.FLOAT64: 'DBL_EPSILON'}}


def _const_data(expr, dtype):
    if dtype in (lang.FLOAT16, lang.FLOAT32):
        return expr.float_data
    if dtype == lang.FLOAT64:
        return expr.double_data
    if dtype in (lang.INT8, lang.INT16, lang.INT32):
        return expr.sint32_data
    if dtype == lang.INT64:
        return expr.sint64_data
    if dtype in (lang.UINT8, lang.UINT16, lang.UINT32):
        return expr.uint32_data
    return expr.uint64_data


def _literal(value):
    """Python's str() of an int or float, which is what the reference pastes into the C text."""
    if isinstance(value, float):
        if value != value:
            return 'NAN'
        if value in (float('inf'), float('-inf')):
            return 'INFINITY' if value > 0 else '-INFINITY'
        return str(float(value))
    return str(int(value))


def _binary_text(code, dtype, a, b):
    if code == lang.MIN:
        return '(((' + a + ')<(' + b + '))?(' + a + '):(' + b + '))'
    if code == lang.MAX:
        return '(((' + a + ')>(' + b + '))?(' + a + '):(' + b + '))'
    if code == lang.POW:
        return ('powf(' if dtype == lang.FLOAT32 else 'pow(') + a + ',' + b + ')'
    if code == lang.ATAN2:
        return ('atan2f(' if dtype == lang.FLOAT32 else 'atan2(') + a + ',' + b + ')'
    if code == lang.MODULO and dtype == lang.FLOAT32:
        return 'fmodf(' + a + ',' + b + ')'
    if code == lang.MODULO and dtype == lang.FLOAT64:
        return 'fmod(' + a + ',' + b + ')'
    return '(' + a + ' ' + INFIX[code] + ' ' + b + ')'


def tensor_size(tensor_type):
    size = 1
    for d in tensor_type.shape:
        size *= d
    return size


def emit_body(dag):
    """Return (list of C statements, input exprs by io_index, output exprs by io_index, num_workers)."""
    names = []
    inputs = {}
    outputs = {}
    stmts = []
    for n, expr in enumerate(dag.expressions):
        ops = dag.references[n].operand_indices
        code = expr.code
        name = 'e' + str(n)
        stmt = None
        if code == lang.INPUT:
            name = '(*in' + str(expr.io_index) + ')'
            inputs[expr.io_index] = expr
        elif code == lang.OUTPUT:
            name = '(*out' + str(expr.io_index) + ')'
            outputs[expr.io_index] = expr
        elif code == lang.POSITION:
            name = 'position'
            shape = list(expr.uint32_data)
            block = [1]
            for dim in range(len(shape) - 1, 0, -1):
                block.append(block[-1] * shape[dim])
            block.reverse()
            vals = []
            remainder = 'worker_index'
            for cur_block in block:
                vals.append('(' + remainder + ')/' + str(cur_block))
                remainder = remainder + ' % ' + str(cur_block)
            stmt = 'const uint32_t position[' + str(len(shape)) + '] = {' + ', '.join(vals) + '};'
        elif code == lang.CONST_SCALAR:
            name = _literal(_const_data(expr, expr.dtype)[0])
        elif code == lang.CONST_TENSOR:
            data = _const_data(expr, expr.tensor_type.dtype)
            name = '{' + ', '.join(_literal(v) for v in data) + '}'
        elif code in LIMITS:
            name = LIMITS[code][expr.dtype]
        elif code in (lang.VARIABLE, lang.CAST):
            stmt = CTYPE[expr.dtype] + ' ' + name + ' = ' + names[ops[0]] + ';'
        elif code == lang.TENSOR:
            stmt = CTYPE[expr.tensor_type.dtype] + ' ' + name + '[' + str(tensor_size(expr.tensor_type)) + '] = ' + \
                names[ops[0]] + ';'
        elif code == lang.ASSIGN_VARIABLE:
            stmt = names[ops[0]] + ' = ' + names[ops[1]] + ';'
        elif code == lang.ASSIGN_TENSOR:
            stmt = names[ops[0]] + '[' + names[ops[1]] + '] = ' + names[ops[2]] + ';'
        elif code == lang.READ_TENSOR:
            stmt = CTYPE[expr.dtype] + ' ' + name + ' = ' + names[ops[0]] + '[' + names[ops[1]] + '];'
        elif code == lang.RANGE:
            i, start, stop, step = (names[o] for o in ops)
            stmt = 'for(' + i + ' = ' + start + '; ((' + i + ' < ' + stop + ')&&(' + step + '>0)) || ((' + \
                i + ' > ' + stop + ')&&(' + step + '<0)); ' + i + '+=' + step + '){'
        elif code == lang.ENDRANGE or code == lang.ENDIF:
            stmt = '}'
        elif code == lang.IF:
            stmt = 'if(' + names[ops[0]] + '){'
        elif code == lang.ELSEIF:
            stmt = '}\nelse if(' + names[ops[0]] + '){'
        elif code == lang.ELSE:
            stmt = '}\nelse{'
        elif code in UNARY:
            stmt = CTYPE[expr.dtype] + ' ' + name + ' = ' + UNARY[code][expr.dtype] + '(' + names[ops[0]] + ');'
        elif code in INFIX or code in (lang.MIN, lang.MAX, lang.POW, lang.ATAN2):
            stmt = CTYPE[expr.dtype] + ' ' + name + ' = ' + \
                _binary_text(code, expr.dtype, names[ops[0]], names[ops[1]]) + ';'
        else:
            raise NotImplementedError('expression code ' + str(code))
        names.append(name)
        if stmt is not None:
            stmts.append(stmt)

    num_workers = 1
    for d in dag.workgroup_shape:
        num_workers *= d
    return stmts, inputs, outputs, num_workers


PROLOGUE = """//Generated Code (test oracle)
#include <stdint.h>
#include <stdlib.h>
#include <math.h>
#include <cfloat>

typedef long long int int64_tf;
typedef struct { void* data; int32_t dtype; uint64_t len; } ovl_tensor;

//aliases for integer absolute values for ints < 32 bits in size
#define abs_8(x) abs(x);
#define abs_16(x) abs(x);
"""


def emit_cpp(dag, function_name):
    """
    C++ source of one operator: the worker function ``<function_name>`` and the exported entry
    ``<function_name>_generic_cpp(in, n_in, out, n_out, num_threads, thread_index, err)``.
    """
    stmts, inputs, outputs, num_workers = emit_body(dag)
    num_inputs = len(inputs)
    num_outputs = len(outputs)

    args = []
    for i in range(num_inputs):
        tt = inputs[i].tensor_type
        args.append('const ' + CTYPE[tt.dtype] + ' (*in' + str(i) + ')[' + str(tensor_size(tt)) + ']')
    for i in range(num_outputs):
        tt = outputs[i].tensor_type
        args.append(CTYPE[tt.dtype] + ' (*out' + str(i) + ')[' + str(tensor_size(tt)) + ']')

    src = [PROLOGUE]
    src.append('void ' + function_name + '(' + ', '.join(args) + ',')
    src.append('                      uint32_t block_size, uint32_t thread_index){')
    src.append('    uint32_t start = thread_index * block_size;')
    src.append('    uint32_t end = start + block_size;')
    src.append('    if (end > ' + str(num_workers) + ') end = ' + str(num_workers) + ';')
    src.append('    for(uint32_t worker_index=start; worker_index < end; worker_index++){')
    for stmt in stmts:
        src.append('        ' + stmt)
    src.append('    }')
    src.append('}')
    src.append('')
    src.append('extern "C"')
    src.append('void ' + function_name + '_generic_cpp(const ovl_tensor* inputs, uint32_t num_inputs,')
    src.append('        ovl_tensor* outputs, uint32_t num_outputs,')
    src.append('        uint32_t num_threads, uint32_t thread_index, uint16_t* err){')
    src.append('    //check that the number of inputs and outputs is correct')
    src.append('    if(num_inputs != ' + str(num_inputs) + '){ *err = 1; return; }')
    src.append('    if(num_outputs != ' + str(num_outputs) + '){ *err = 1; return; }')
    call_args = []
    for kind, table, const in (('in', inputs, 'const '), ('out', outputs, '')):
        for i in range(len(table)):
            tt = table[i].tensor_type
            ctype = CTYPE[tt.dtype]
            size = str(tensor_size(tt))
            var = kind + str(i)
            arr = kind + 'puts[' + str(i) + ']'
            src.append('    if(' + arr + '.len != ' + size + ') { *err = 1; return; }')
            src.append('    if(' + arr + '.dtype != ' + str(tt.dtype) + ') { *err = 1; return; }')
            src.append('    ' + const + ctype + ' (*' + var + ')[' + size + '] = (' + const + ctype + ' (*)[' + size +
                       '])' + arr + '.data;')
            call_args.append(var)
    src.append('    uint32_t block_size = ' + str(num_workers) + ' / num_threads;')
    src.append('    if(' + str(num_workers) + ' % num_threads > 0) block_size += 1;')
    src.append('    return ' + function_name + '(' + ', '.join(call_args) + ', block_size, thread_index);')
    src.append('}')
    return '\n'.join(src) + '\n'
