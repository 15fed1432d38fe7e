"""Writes reference_vectors.json: the inputs and expected outputs that the reference's own tests hold, as data.

Every case is transcribed by hand from the reference test it cites (`cite` = file:lines under the reference tree);
nothing of the reference is imported, run or read by this script. Where a reference test computes its expectation
with a libm call (`std::log(x)` ...), the case carries `expected_expr` naming that function instead of numbers.
A few expected arrays that the reference spells out in full are rebuilt here from their closed form and asserted
against spot values copied from the reference file, so a transcription slip fails here and not in a parity test.

Run from the repository root:  python tests/golden/make_vectors.py
"""
import json
seq96 = [float(i) for i in range(1, 97)]
k3 = [1.0, 0.0, -1.0] * 9
cases = []
def case(name, cite, op, inputs, expected, **kw):
    cases.append(dict(name=name, cite=cite, op=op, inputs=inputs, expected=expected, **kw))
def t(shape, data, dtype="float32", transpose=None):
    d = dict(dtype=dtype, shape=shape, data=data)
    if transpose: d["transpose"] = transpose
    return d
# ---- matmul
case("matmul_batched", "tests/cpu/test-matmul.cpp:12-40", "matmul",
     [t([1,2,2,2],[1,2,3,4,5,6,7,8]), t([1,2,2,2],[9,8,7,6,5,4,3,2])], t([1,2,2,2],[23,20,55,48,43,32,59,44]))
case("matmul_second_transposed", "tests/cpu/test-matmul.cpp:42-64", "matmul",
     [t([2,3],[1,2,3,4,5,6]), t([2,3],[7,8,9,10,11,12], transpose=[-1,-2])], t([2,2],[50,68,122,167]))
case("matmul_both_transposed", "tests/cpu/test-matmul.cpp:66-89", "matmul",
     [t([3,2],[1,4,2,5,3,6], transpose=[-1,-2]), t([2,3],[7,8,9,10,11,12], transpose=[-1,-2])], t([2,2],[50,68,122,167]))
case("matmul_rank4_second_transposed", "tests/cpu/test-matmul.cpp:91-138", "matmul",
     [t([2,2,2,4],[1,2,3,4,5,6,7,8]*4),
      t([2,2,3,4],list(range(1,25))+[1,0,1,0,0,1,0,1,1,1,1,1,2,2,2,2,3,3,3,3,4,4,4,4], transpose=[-1,-2])],
     t([2,2,2,3],[30,70,110,70,174,278,150,190,230,382,486,590,4,6,10,12,14,26,20,30,40,52,78,104]))
exp = []
X = seq96; Y = [float(i) for i in range(1,25)]
for b in range(6):
    for i in range(4):
        for j in range(6):
            exp.append(sum(X[b*16+i*4+k]*Y[j*4+k] for k in range(4)))
# spot values copied from the reference file, checked against the closed form above
assert exp[0]==30 and exp[5]==230 and exp[23]==1310 and exp[143]==8510 and exp[72]==510 and exp[104]==2966 and exp[100]==4926
case("matmul_rank4_rank2_strided_transposed", "tests/cpu/test-matmul.cpp:140-238", "matmul",
     [t([2,3,4,4],seq96), t([6,4],Y, transpose=[-1,-2])], t([2,3,4,6],exp))
# ---- conv2d
i9=[1,2,3,4,5,6,7,8,9]
case("conv2d_simple", "tests/cpu/test-convolutions.cpp:130-151", "conv2d", [t([1,1,3,3],i9), t([1,1,2,2],[1,0,0,-1])], t([1,1,2,2],[-4]*4), stride=[1,1], padding=[0,0])
case("conv2d_stride2", "tests/cpu/test-convolutions.cpp:153-174", "conv2d", [t([1,1,4,4],list(range(1,17))), t([1,1,2,2],[1,0,0,-1])], t([1,1,2,2],[-5]*4), stride=[2,2], padding=[0,0])
case("conv2d_kernel1x1", "tests/cpu/test-convolutions.cpp:233-253", "conv2d", [t([1,1,3,3],i9), t([1,1,1,1],[2])], t([1,1,3,3],[2,4,6,8,10,12,14,16,18]), stride=[1,1], padding=[0,0])
big=[-120,-12,-12,126,-198,-18,-18,207,-234,-18,-18,243,-168,-12,-12,174,-408,-12,-12,414,-630,-18,-18,639,-666,-18,-18,675,-456,-12,-12,462]
case("conv2d_big", "tests/cpu/test-convolutions.cpp:255-344", "conv2d", [t([2,3,4,4],seq96), t([1,3,3,3],k3)], t([2,1,4,4],big), stride=[1,1], padding=[1,1])
case("conv2d_big_biased", "tests/cpu/test-convolutions.cpp:346-432", "conv2d", [t([2,3,4,4],seq96), t([1,3,3,3],k3), t([1],[10])], t([2,1,4,4],[v+10 for v in big]), stride=[1,1], padding=[1,1])
b0=[-110,-2,-2,136,-188,-8,-8,217,-224,-8,-8,253,-158,-2,-2,184]
b0n=[115,7,7,-131,193,13,13,-212,229,13,13,-248,163,7,7,-179]
b1=[-398,-2,-2,424,-620,-8,-8,649,-656,-8,-8,685,-446,-2,-2,472]
b1n=[403,7,7,-419,625,13,13,-644,661,13,13,-680,451,7,7,-467]
assert b0==[v+10 for v in big[:16]] and b1==[v+10 for v in big[16:]]
case("conv2d_big_biased_two_out_channels", "tests/cpu/test-convolutions.cpp:434-490", "conv2d",
     [t([2,3,4,4],seq96), t([2,3,3,3],k3+[-v for v in k3]), t([2],[10,-5])], t([2,2,4,4],b0+b0n+b1+b1n), stride=[1,1], padding=[1,1])
# ---- elementwise
A=[0,1,2,3,4,5]; B=[0,10,20,30,40,50,60,70,80,90,100,110]
case("neg", "tests/cpu/test-operations.cpp:11-29", "neg", [t([3,3],list(range(9,18)))], t([3,3],[-v for v in range(9,18)]))
case("add_broadcast", "tests/cpu/test-operations.cpp:31-57", "add", [t([2,1,3],A), t([1,4,3],B)],
     t([2,4,3],[0,11,22,30,41,52,60,71,82,90,101,112,3,14,25,33,44,55,63,74,85,93,104,115]))
case("mul_broadcast", "tests/cpu/test-operations.cpp:59-85", "mul", [t([2,1,3],A), t([1,4,3],B)],
     t([2,4,3],[0,10,40,0,40,100,0,70,160,0,100,220,0,40,100,90,160,250,180,280,400,270,400,550]))
case("sub_broadcast", "tests/cpu/test-operations.cpp:87-113", "sub", [t([2,1,3],A), t([1,4,3],B)],
     t([2,4,3],[0,-9,-18,-30,-39,-48,-60,-69,-78,-90,-99,-108,3,-6,-15,-27,-36,-45,-57,-66,-75,-87,-96,-105]))
case("complex_mul", "tests/cpu/test-operations.cpp:115-134", "complex_mul", [t([2,2],[1,6,2,3]), t([2,2],[2,1,1.5,3.14])], t([2,2],[-4.0,13.0,-6.42,10.78]), rtol=1e-3)
case("pow_broadcast", "tests/cpu/test-operations.cpp:136-160", "pow", [t([2,1,3],A), t([1,4,3],B)], None, expected_expr="pow")
case("broadcast_multiply_add", "tests/cpu/test-operations.cpp:162-181", "mul_add",
     [t([2,3],[-1.22474,0,1.22474,-1.22474,0,1.22474]), t([3],[0.5,1.0,1.5]), t([3],[0.0,0.1,0.2])],
     t([2,3],[-0.61237,0.1,2.03711,-0.61237,0.1,2.03711]), rtol=1e-5)
for fn in ["log","exp","sqrt","sin","cos","tan","sinh","cosh","tanh"]:
    case("fn_"+fn, "tests/cpu/test-functions.cpp", fn, [t([2,3],[1,2,3,4,5,6])], None, expected_expr=fn)
case("fn_rsqrt", "tests/cpu/test-functions.cpp:52-65", "rsqrt", [t([2,3],[1,2,3,4,5,6])], None, expected_expr="rsqrt", eps=1e-6)
case("fn_abs", "tests/cpu/test-functions.cpp:67-76", "abs", [t([2,3],[-1,-2,-3,-4,-5,-6])], t([2,3],[1,2,3,4,5,6]))
# ---- reductions
x1=[3,5,4,1,5,9,2]
x2=[3,5,4,1,5,9,2,7,6,2,8,4]
case("argmax_1d", "tests/cpu/test-reductions.cpp:11-19", "argmax", [t([7],x1)], t([],[5],"int64"), axis=0)
case("argmin_1d", "tests/cpu/test-reductions.cpp:11-19", "argmin", [t([7],x1)], t([],[3],"int64"), axis=0)
case("argmax_2d_last", "tests/cpu/test-reductions.cpp:21-38", "argmax", [t([3,4],x2)], t([3],[1,1,2],"int64"), axis=-1)
case("argmin_2d_last", "tests/cpu/test-reductions.cpp:21-38", "argmin", [t([3,4],x2)], t([3],[3,2,1],"int64"), axis=-1)
case("argmax_2d_axis0", "tests/cpu/test-reductions.cpp:40-60", "argmax", [t([3,4],x2)], t([4],[2,1,2,1],"int64"), axis=0)
case("argmin_2d_axis0", "tests/cpu/test-reductions.cpp:40-60", "argmin", [t([3,4],x2)], t([4],[0,2,1,0],"int64"), axis=0)
case("sum_2d_keepdim", "tests/cpu/test-reductions.cpp:62-73", "sum", [t([2,3],[1,2,3,4,5,6])], t([2,1],[6,15]), axis=1, keepdim=True)
case("mean_2d_axis0", "tests/cpu/test-reductions.cpp:75-87", "mean", [t([2,3],[1,2,3,4,5,6])], t([3],[2.5,3.5,4.5]), axis=0)
case("sum_1d", "tests/cpu/test-reductions.cpp:89-97", "sum", [t([5],[10,20,30,40,50])], t([],[150]), axis=-1)
case("mean_1d", "tests/cpu/test-reductions.cpp:89-97", "mean", [t([5],[10,20,30,40,50])], t([],[30]), axis=-1)
case("sum_1d_keepdim", "tests/cpu/test-reductions.cpp:99-109", "sum", [t([5],[10,20,30,40,50])], t([1],[150]), axis=0, keepdim=True)
case("mean_1d_keepdim", "tests/cpu/test-reductions.cpp:99-109", "mean", [t([5],[10,20,30,40,50])], t([1],[30]), axis=0, keepdim=True)
case("sum_2d_last_keepdim", "tests/cpu/test-reductions.cpp:111-127", "sum", [t([2,4],list(range(1,9)))], t([2,1],[10,26]), axis=-1, keepdim=True)
case("mean_2d_last_keepdim", "tests/cpu/test-reductions.cpp:111-127", "mean", [t([2,4],list(range(1,9)))], t([2,1],[2.5,6.5]), axis=-1, keepdim=True)
case("sum_3d_last_keepdim", "tests/cpu/test-reductions.cpp:129-160", "sum", [t([2,3,4],list(range(1,25)))], t([2,3,1],[10,26,42,58,74,90]), axis=-1, keepdim=True)
case("mean_3d_last_keepdim", "tests/cpu/test-reductions.cpp:129-160", "mean", [t([2,3,4],list(range(1,25)))], t([2,3,1],[2.5,6.5,10.5,14.5,18.5,22.5]), axis=-1, keepdim=True)
case("mean_of_squares", "tests/cpu/test-reductions.cpp:162-175", "mean_sq", [t([2,2,3],[1,2,3,4,5,6,-1,-2,-3,0.5,1.0,1.5])], t([2,2],[4.6667,25.6667,4.6667,1.1667]), axis=-1, atol=1e-3)
# ---- complex
case("polar", "tests/cpu/test-complex.cpp:40-62", "polar", [t([2,2],[1,6,2,3]), t([2,2],[2,1,1.5,3.14])],
     t([2,2,2],[-0.416147,0.909297,3.24181,5.04883,0.141474,1.99499,-3.0,0.00477764]), rtol=1e-5, atol=1e-5)
freq=[1.0,0.0,1.0,0.0,1.0,0.0, 0.5403,0.8415,0.9989,0.0464,1.0,0.0022, -0.4161,0.9093,0.9957,0.0927,1.0,0.0043, -0.99,0.1411,0.9903,0.1388,1.0,0.0065,
      -0.6536,-0.7568,0.9828,0.1846,1.0,0.0086, 0.2837,-0.9589,0.9732,0.23,0.9999,0.0108, 0.9602,-0.2794,0.9615,0.2749,0.9999,0.0129, 0.7539,0.657,0.9477,0.3192,0.9999,0.0151]
case("llama_freq_cis", "tests/cpu/test-complex.cpp:64-108", "freq_cis", [], t([8,3,2],freq,"float64"), model_dimension=6, sequence_length=8, theta=10000.0, rtol=0.1, atol=0.1)
# ---- 16-bit conversions (tests/test-types.cpp:45-166) and known answers of 16-bit native accumulation (sums of ones stall at 2048)
case("half_bits", "tests/test-types.cpp:45-166", "half_bits", [], None,
     pairs=[[0.0,0x0000],[-0.0,0x8000],[1.0,0x3C00],[-2.0,0xC000],["inf",0x7C00],["-inf",0xFC00],[5.960464477539063e-08,0x0001],[65504.0,0x7BFF],[1e5,0x7C00]])
case("bhalf_bits", "tests/test-types.cpp:45-166", "bhalf_bits", [], None,
     pairs=[[0.0,0x0000],[-0.0,0x8000],[1.0,0x3F80],[-2.0,0xC000],["inf",0x7F80],["-inf",0xFF80]])
case("native_f16_dot_of_ones", "src/cpu/matmul.cpp:32-36 run on 4096 ones", "native_dot", [], None, length=4096, expected_value=2048.0)
case("native_f16_sum_of_ones", "src/cpu/argred.cpp:32-35 run on 4096 ones", "native_sum", [], None, length=4096, expected_value=2048.0)
case("mixed_f16_f32_dot_of_ones", "src/cpu/matmul.cpp:213-214 run on 4096 ones", "wide_dot", [], None, length=4096, expected_value=4096.0)
# ---- repeats, conv1d, concatenation, outer product
def tv(shape, data, **view):
    return dict(dtype="float32", shape=shape, data=data, **view)
r22 = tv([2,2],[1,2,3,4])
case("repeat_axis0", "tests/cpu/test-repeats.cpp:9-29", "repeat", [r22], t([4,2],[1,2,1,2,3,4,3,4]), repeats=2, axis=0)
case("repeat_axis1", "tests/cpu/test-repeats.cpp:32-53", "repeat", [r22], t([2,4],[1,1,2,2,3,3,4,4]), repeats=2, axis=1)
case("repeat_after_permute", "tests/cpu/test-repeats.cpp:84-148", "repeat", [tv([2,2,3],list(range(1,13)),permute=[2,0,1])],
     t([6,2,2],[1,4,7,10]*2+[2,5,8,11]*2+[3,6,9,12]*2), repeats=2, axis=0)
d3=[1,0,-1]
case("conv1d_simple", "tests/cpu/test-convolutions.cpp:13-27", "conv1d", [t([1,1,5],[1,2,3,4,5]), t([1,1,3],d3)], t([1,1,3],[-2,-2,-2]), stride=1, padding=0)
case("conv1d_stride2", "tests/cpu/test-convolutions.cpp:29-43", "conv1d", [t([1,1,6],[1,2,3,4,5,6]), t([1,1,3],d3)], t([1,1,2],[-2,-2]), stride=2, padding=0)
case("conv1d_padding1", "tests/cpu/test-convolutions.cpp:45-58", "conv1d", [t([1,1,3],[1,2,3]), t([1,1,2],[1,-1])], t([1,1,4],[-1,-1,-1,3]), stride=1, padding=1)
case("conv1d_multi_channel_input", "tests/cpu/test-convolutions.cpp:60-83", "conv1d", [t([1,2,4],list(range(1,9))), t([1,2,3],[1]*6)], t([1,1,2],[24,30]), stride=1, padding=0)
case("conv1d_kernel_1", "tests/cpu/test-convolutions.cpp:85-99", "conv1d", [t([1,1,4],[1,2,3,4]), t([1,1,1],[2])], t([1,1,4],[2,4,6,8]), stride=1, padding=0)
case("conv1d_multi_output_channels", "tests/cpu/test-convolutions.cpp:101-133", "conv1d", [t([1,1,5],[1,2,3,4,5]), t([2,1,3],d3+[0,1,0])],
     t([1,2,3],[-2,-2,-2,2,3,4]), stride=1, padding=0)
case("concat_axis0", "tests/cpu/test-concat.cpp:8-29", "concat", [r22, t([3,2],[5,6,7,8,9,10])], t([5,2],list(range(1,11))), axis=0)
case("concat_axis1", "tests/cpu/test-concat.cpp:31-49", "concat", [r22, t([2,3],[5,6,7,8,9,10])], t([2,5],[1,2,5,6,7,3,4,8,9,10]), axis=1)
case("concat_expanded_with_transposed", "tests/cpu/test-concat.cpp:51-84", "concat",
     [tv([1,1,3],[100,200,300],expand=[2,-1,-1]), tv([2,3,4],list(range(1,25)),transpose=[1,2])],
     t([2,5,3],[100,200,300,1,5,9,2,6,10,3,7,11,4,8,12,100,200,300,13,17,21,14,18,22,15,19,23,16,20,24]), axis=1)
case("outer_vectors", "tests/cpu/test-outer-product.cpp:7-23", "outer", [t([2],[1.5,-2.0]), t([3],[4.0,0.0,-1.0])], t([2,3],[6.0,0.0,-1.5,-8.0,0.0,2.0]))
# ---- strided views copied into contiguous tensors (reshape of a transposed tensor, reads of a permuted one)
tr = [1.0 + b*48 + c*16 + i*4 + j for b in range(2) for i in range(4) for c in range(3) for j in range(4)]
# rows copied from the reference file, checked against the closed form above
assert tr[0:12] == [1,2,3,4,17,18,19,20,33,34,35,36] and tr[36:48] == [13,14,15,16,29,30,31,32,45,46,47,48]
assert tr[48:60] == [49,50,51,52,65,66,67,68,81,82,83,84] and tr[84:96] == [61,62,63,64,77,78,79,80,93,94,95,96]
case("repack_transposed_then_reshaped", "tests/cpu/test-non-contiguous.cpp:12-76", "repack", [tv([2,3,4,4],seq96,transpose=[1,2])], t([2,4,3,4],tr))
pm = [1.0 + j*12 + k*4 + i for i in range(4) for j in range(2) for k in range(3)]      # the formula the reference test states
case("repack_permuted_234_to_423", "tests/cpu/test-repeats.cpp:55-81", "repack", [tv([2,3,4],[float(v) for v in range(1,25)],permute=[2,0,1])], t([4,2,3],pm))
# ---- complex views
case("complexify_then_realify", "tests/cpu/test-complex.cpp:17-38", "complex_roundtrip", [t([2,2],[1,0,2,3])], t([2,2],[1,0,2,3]))
freqs = [1.0,0.0, 1.0,0.0, 1.0,0.0,  0.5403,0.8415, 0.9989,0.0464, 1.0,0.0022,  -0.4161,0.9093, 0.9957,0.0927, 1.0,0.0043,
         -0.9900,0.1411, 0.9903,0.1388, 1.0,0.0065,  -0.6536,-0.7568, 0.9828,0.1846, 1.0,0.0086,  0.2837,-0.9589, 0.9732,0.2300, 0.9999,0.0108,
         0.9602,-0.2794, 0.9615,0.2749, 0.9999,0.0129,  0.7539,0.6570, 0.9477,0.3192, 0.9999,0.0151]
rot = [1.0,2.0,-1.7451,4.6857,-7.5363,2.0499,-8.0588,-6.9323,1.6856,-13.3472,14.6275,-7.1435,16.3942,9.8106,0.7965,21.9174,
       17.0,18.0,18.0511,20.8596,18.8703,23.8521,19.4457,26.9596,19.7704,30.1678,19.8364,33.4596,19.6365,36.8171,19.1643,40.2216,
       33.0,34.0,34.9208,36.0770,36.8366,38.1591,38.7400,40.2535,40.6388,42.3526,42.5205,44.4600,44.4021,46.5759,46.2705,48.7049]
# the sequence as pairs times the frequencies [8 positions... of 3 rows][2], complexified and transposed to [3, 8]: rotary embedding by complex product
case("rotary_embedding_by_complex_product", "tests/cpu/test-complex.cpp:110-157", "complex_mul",
     [t([1,1,3,8,2],[float(v) for v in range(1,49)]), tv([8,3,2],freqs,transpose=[0,1])], t([1,1,3,8,2],rot), rtol=1e-4, atol=1e-3)
# ---- assignment of a tensor to a slice (a strided copy into existing memory)
assigned = list(freqs)
assigned[2*6:5*6] = [1.0] * 18
case("assign_tensor_to_slice", "tests/cpu/test-views.cpp:392-419", "assign_rows", [t([8,3,2],freqs), t([3,3,2],[1.0]*18)], t([8,3,2],assigned), rows=[2,5])
json.dump(dict(note="Inputs and expected outputs held by the reference's own tests (tests/cpu/*.cpp, tests/test-types.cpp), transcribed as data; "
               "'cite' names the reference file and lines. Cases with expected_expr compare against the same libm function the reference test evaluates.",
               cases=cases), open("tests/golden/reference_vectors.json","w"), indent=0)
print(len(cases))
