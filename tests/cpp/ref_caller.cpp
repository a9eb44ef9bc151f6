// A caller written only against the reference's public class API (Msnhnet/Msnhnet.h: NetBuilder, YoloBox, Exception, TimeUtil), in the
// shape of its own examples (examples/deeplearning/yolov3_gpu/yolov3_gpu.cpp, classify_gpu/classify_gpu.cpp).  The tests compile it
// against msnhnet_amd/host/include, link libMsnhnet.so and run it on the GPU: the class-level drop-in claim, exercised as C++.
//
//   ref_caller classify|yolo <graph.msnhnet> <weights.msnhbin> <input.f32> <output.f32> [fp16]
//
// input: one CHW float32 image as raw bytes; output: the logits, or rows of 7 floats (x y w h conf bestClsConf bestClsIdx).
#include <cstdio>
#include <fstream>
#include <iostream>
#include <string>
#include <vector>
#include "Msnhnet/Msnhnet.h"

int main(int argc, char **argv)
{
    if (argc < 6)
    {
        std::cout << "usage: ref_caller classify|yolo graph weights input output [fp16]" << std::endl;
        return 2;
    }
    const std::string mode = argv[1];
    try
    {
        Msnhnet::NetBuilder msnhNet;
        Msnhnet::NetBuilder::setOnlyGpu(true);
        Msnhnet::NetBuilder::setUseFp16(argc > 6 && std::string(argv[6]) == "fp16");
        msnhNet.buildNetFromMsnhNet(argv[2]);
        std::cout << msnhNet.getLayerDetail();
        msnhNet.loadWeightsFromMsnhBin(argv[3]);
        Msnhnet::Point2I inSize = msnhNet.getInputSize();
        std::vector<float> img(static_cast<size_t>(inSize.x) * inSize.y * msnhNet.getInputChannel());
        std::ifstream in(argv[4], std::ios::binary);
        in.read(reinterpret_cast<char *>(img.data()), static_cast<std::streamsize>(img.size() * sizeof(float)));
        if (!in) { std::cout << "short input file" << std::endl; return 3; }

        std::vector<float> out;
        for (size_t i = 0; i < 3; i++)
        {
            auto st = Msnhnet::TimeUtil::startRecord();
            if (mode == "yolo")
            {
                std::vector<std::vector<Msnhnet::YoloBox>> result = msnhNet.runYoloGPU(img);
                out.clear();
                for (const Msnhnet::YoloBox &b : result[0])
                {
                    const float row[7] = {b.xywhBox.x, b.xywhBox.y, b.xywhBox.w, b.xywhBox.h, b.conf, b.bestClsConf, static_cast<float>(b.bestClsIdx)};
                    out.insert(out.end(), row, row + 7);
                }
            }
            else
                out = msnhNet.runClassifyGPU(img);
            std::cout << "time  : " << Msnhnet::TimeUtil::getElapsedTime(st) << "ms  (device side " << msnhNet.getGpuInferenceTime() << " ms)" << std::endl;
        }
        std::ofstream o(argv[5], std::ios::binary);
        o.write(reinterpret_cast<const char *>(out.data()), static_cast<std::streamsize>(out.size() * sizeof(float)));

        // the CPU entry point exists and refuses, with the reference's message for a GPU-only build
        try { msnhNet.runClassify(img); return 4; }
        catch (Msnhnet::Exception ex) { std::cout << "cpu: " << ex.what() << std::endl; }
    }
    catch (Msnhnet::Exception ex)
    {
        std::cout << ex.what() << " " << ex.getErrFile() << " " << ex.getErrLine() << " " << ex.getErrFun() << std::endl;
        return 1;
    }
    return 0;
}
