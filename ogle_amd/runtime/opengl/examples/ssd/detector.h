// SSD detector driver: runs the graph, then decode + score filter and top-k + NMS
// on the device (or, with device_nms off, top-k + NMS on the host as the reference
// does); one readback of the final lists.  Counterpart of
// ogl_runtime/opengl/examples/ssd/detector.{h,cc} without the OpenCV image I/O:
// the caller passes preprocessed float images (NHWC) and the size the boxes are
// scaled to.  Unlike the reference, which post-processes the first image only
// (detector.cc:184), every image of the batch is handled.
#ifndef OPENGL_EXAMPLES_SSD_DETECTOR_H_
#define OPENGL_EXAMPLES_SSD_DETECTOR_H_
#include <memory>
#include <string>
#include <vector>

#include "opengl/core/types.h"

namespace opengl {

// Integer rectangle with cv::Rect's fields.
struct Rect {
  int x = 0, y = 0, width = 0, height = 0;
};

// examples/ssd/common.h:29-45 of the reference.
struct BoxInfo {
  Rect box;
  float score = 0.f;
  float cx = 0.f, cy = 0.f;
  float width = 0.f, height = 0.f;
  int class_name = 0;
  int index = 0;  // prior index
};

struct DetectorOptions {
  string model_name;
  int input_width = 0;
  int input_height = 0;
  float nms_threshold = 0.45f;
  float score_threshold = 0.3f;
  int topk = 100;
  // Top-k + NMS on the device (ogle_hip_ssd_topk_nms) instead of the host loop of
  // detector.cc:114-148; same results, and only the final lists are read back.
  // Needs topk <= 1024 and at most 8192 priors; the host path is used otherwise.
  bool device_nms = true;
  std::vector<float> variances = {0.1f, 0.1f, 0.2f, 0.2f};
  TensorNameList input_names = {"input"};
  TensorNameList output_names = {"cls_logits", "box_preds", "anchors"};
};

class FBOSession;

class Detector {
 public:
  static std::unique_ptr<Detector> Create(const DetectorOptions& options);
  // Wraps a session the caller already loaded (not owned).
  static std::unique_ptr<Detector> Create(FBOSession* session, const DetectorOptions& options);
  ~Detector();

  // images: host NHWC float tensor, already mean-subtracted and resized
  // (Preprocess, detector.cc:99-109, is image I/O and stays with the caller).
  // Boxes are scaled to raw_width x raw_height.  One vector per image.
  void Detect(const Tensor* images, int raw_width, int raw_height,
              std::vector<std::vector<BoxInfo>>* final_boxes);

  // The stages, as in the reference.
  void Run(const Tensor* images);
  void LoadToOutputTensors(const TensorNameList& names, int raw_width, int raw_height);
  // The two halves of LoadToOutputTensors: the device launch (asynchronous, buffers
  // allocated on first use) and the readback of its compacted results (synchronises).
  // lists_in_place: skip the compaction launch and leave every prior's record at its own
  // slot (kept prior index or -1); only EnqueueTopkNms can read such lists.
  void EnqueuePostprocess(const TensorNameList& names, int raw_width, int raw_height,
                          bool lists_in_place = false);
  void Readback();
  // Device top-k + NMS over what EnqueuePostprocess left on the device
  // (asynchronous), and the readback of its final lists (synchronises).
  void EnqueueTopkNms();
  void ReadbackFinal(std::vector<std::vector<BoxInfo>>* final_boxes);
  // Pipelined readback: once enabled, EnqueueTopkNms is followed on the stream by ONE
  // asynchronous copy of the final lists (they are one device block: the counts, then at most
  // topk records per image) into page-locked host memory owned by the detector.  Recorded
  // into a captured pass it replays with it, so the host only waits for an event after the
  // pass (not for the stream) and then reads the lists with FinalFromHostCopy, while later
  // passes are already enqueued.  The copy lands in the same memory every pass: read it
  // before the detector's next pass is launched.
  void EnableHostCopy();
  bool host_copy_enabled() const { return final_host_ != nullptr; }
  void FinalFromHostCopy(std::vector<std::vector<BoxInfo>>* final_boxes) const;
  bool UsesDeviceNms() const;
  // Everything Detect does on the device after the network (asynchronous): the score
  // filter, and with device top-k + NMS that launch too (ReadbackFinal fetches its
  // lists; otherwise Readback + HostTopkNms finish on the host).
  void EnqueueDetect(const TensorNameList& names, int raw_width, int raw_height);
  // The reference's host loop over what Readback() fetched: GenerateBoxInfo, GetTopK,
  // NMS per image.
  void HostTopkNms(std::vector<std::vector<BoxInfo>>* final_boxes) const;
  void GenerateBoxInfo(int image, std::vector<BoxInfo>* box_infos) const;
  static void GetTopK(std::vector<BoxInfo>& input, int top_k);
  static void NMS(std::vector<BoxInfo>& boxes, std::vector<BoxInfo>& boxes_left, float threshold);

  FBOSession* session() const { return session_; }

 private:
  Detector(FBOSession* session, bool owned, const DetectorOptions& options);
  DetectorOptions options_;
  FBOSession* session_;
  bool owns_session_;
  int batch_ = 0, priors_ = 0, classes_ = 0;
  int priors_for_nms_ = 0;       // prior count of the outputs last looked at
  bool lists_in_place_ = false;  // how the last EnqueuePostprocess left the kept lists
  // device results of the fused decode + score filter, and their host copies
  std::unique_ptr<Tensor> boxes_dev_, count_dev_, prior_dev_, class_dev_, score_dev_, box_dev_,
      rect_dev_;
  std::vector<int32_t> count_, prior_, class_, rect_;
  std::vector<float> score_, box_;
  // final lists of the device top-k + NMS: (batch, topk) each
  int final_topk_ = 0;
  // one device block: counts (batch), then prior, class, score (batch x topk each), box and
  // rect (batch x topk x 4 each); 4-byte elements throughout
  std::unique_ptr<Tensor> final_dev_;
  std::vector<int32_t> final_staging_;   // host copy made by ReadbackFinal
  void* final_host_ = nullptr;           // page-locked copy made on the stream (EnableHostCopy)
  bool want_host_copy_ = false;
  size_t FinalWords() const;
  void ParseFinal(const int32_t* block, std::vector<std::vector<BoxInfo>>* final_boxes) const;
};

float iou(const Rect& box0, const Rect& box1);

}  // namespace opengl
#endif  // OPENGL_EXAMPLES_SSD_DETECTOR_H_
