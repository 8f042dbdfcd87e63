"""Records C-ABI launches (split-K product + Kahan fold, batched product, softmax, batched
product, the attention block in one launch, a forward convolution with bias) into a HIP graph through torch and replays it: every replay must give the bits of the
eager run, and new operand values in the same buffers must be picked up.  Run by
tests/test_gpu_concurrency.py in a process of its own; exit code 77 = torch has no GPU."""
import os
import sys

try:
    import torch                      # before the library: the process keeps the first HIP runtime loaded
except ImportError:
    print("torch is not importable")
    sys.exit(77)
if not torch.cuda.is_available():
    print("torch sees no GPU")
    sys.exit(77)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "dragon-alpha-v1.2_amd"))
import dragon_hip as dh               # noqa: E402


def main():
    MM, BMM, RD, AT, CV = dh.Cuda_matMul, dh.Cuda_batchMatMul, dh.Cuda_reduce, dh.Cuda_attention, dh.Cuda_conv3D
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(5)
    N, M, K, GZ = 132, 260, 1000, 4
    A = torch.randint(-3, 4, (N, K), generator=g).float().to(dev)
    B = torch.randint(-3, 4, (K, M), generator=g).float().to(dev)
    C = torch.empty(N, M, device=dev)
    Cbuf = torch.empty(GZ - 1, N, M, device=dev)
    Bt, S, D = 4, 64, 32
    Q = torch.randn(Bt, S, D, generator=g).to(dev)
    Kk = torch.randn(Bt, S, D, generator=g).to(dev)
    V = torch.randn(Bt, S, D, generator=g).to(dev)
    P = torch.empty(Bt, S, S, device=dev)
    O = torch.empty(Bt, S, D, device=dev)
    O2 = torch.empty(Bt, S, D, device=dev)
    X = torch.randint(-3, 4, (4, 9, 8, 16), generator=g).float().to(dev)
    W = torch.randint(-3, 4, (20, 3, 3, 16), generator=g).float().to(dev)
    bias = torch.randint(-3, 4, (20,), generator=g).float().to(dev)
    Y = torch.empty(4, 9, 8, 20, device=dev)

    def work(stream):
        s = [stream]
        MM.matMulSK(s, 1, GZ, A.data_ptr(), B.data_ptr(), C.data_ptr(), Cbuf.data_ptr(), N, M, K)
        MM.SKbuf_summary(stream, Cbuf.data_ptr(), C.data_ptr(), GZ - 1, N * M)
        BMM.batchMatMulT2(s, 1, Q.data_ptr(), Kk.data_ptr(), P.data_ptr(), Bt, S, S, S, D)
        RD.softmax2D(stream, P.data_ptr(), P.data_ptr(), Bt * S, S, S, S, 0.25)
        BMM.batchMatMul(s, 1, P.data_ptr(), V.data_ptr(), O.data_ptr(), Bt, S, D, S, S)
        AT.forward(s, 1, Q.data_ptr(), Kk.data_ptr(), V.data_ptr(), O2.data_ptr(), 1, Bt, S, S, D, D, 0, 0.25)
        CV.conv3D_biased(s, 1, X.data_ptr(), 9, 8, W.data_ptr(), 3, 3, Y.data_ptr(), 9, 8, 4, 16, 20, 1, 1, 1, 1,
                         bias.data_ptr(), Y.numel(), 20)

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        work(side.cuda_stream)                      # eager once: also warms the launcher's caches
    side.synchronize()
    C_eager, O_eager, O2_eager, Y_eager = C.clone(), O.clone(), O2.clone(), Y.clone()
    assert torch.equal(C_eager, A @ B)              # integer operands: exact
    Y_ref = torch.nn.functional.conv2d(X.permute(0, 3, 1, 2).double(), W.permute(0, 3, 1, 2).double(),
                                       bias.double(), padding=1).permute(0, 2, 3, 1).float()
    assert torch.equal(Y_eager, Y_ref)
    assert (O2_eager - O_eager).abs().max().item() <= 2e-6
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        work(torch.cuda.current_stream().cuda_stream)
    for rep in range(3):
        C.fill_(-1.0); O.fill_(-1.0); Cbuf.fill_(-2.0); P.fill_(-3.0); O2.fill_(-4.0); Y.fill_(-5.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(C, C_eager), rep
        assert torch.equal(O, O_eager), rep
        assert torch.equal(O2, O2_eager), rep
        assert torch.equal(Y, Y_ref), rep
    # new operand values in the same buffers: the graph picks them up
    A.copy_(torch.randint(-3, 4, (N, K), generator=g).float())
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(C, A @ B)
    print("graph replay ok")


if __name__ == "__main__":
    main()
