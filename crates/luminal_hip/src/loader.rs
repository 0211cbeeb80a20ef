//! GGUF loader for the HIP backend: what `q8_load` of examples/llama/src/loader.rs:99-165 does for CUDA.
//!
//! The header reader lives here because the example's `gguf` module is not part of the luminal library.  It keeps
//! what the loader needs per tensor (element count, offset, ggml dtype) and skips the metadata values, except for
//! `general.alignment`.
use std::{
    collections::HashMap,
    fs::File,
    io::{Read, Seek, SeekFrom},
    path::Path,
};

use byteorder::{LittleEndian, ReadBytesExt};
use luminal::{op::Function, prelude::*};

use crate::quantized::HipData;

const DEFAULT_ALIGNMENT: u64 = 32;
const GGML_F32: u32 = 0;
const GGML_Q8_0: u32 = 8;

struct TensorInfo {
    n_elements: usize,
    offset: u64,
    dtype: u32,
}

struct Header {
    tensors: HashMap<String, TensorInfo>,
    data_offset: u64,
}

struct Reader<R> {
    inner: R,
    wide: bool, // versions 2 and 3 hold 64-bit counts and lengths, version 1 32-bit ones
}

impl<R: Read + Seek> Reader<R> {
    fn size(&mut self) -> u64 {
        if self.wide {
            self.inner.read_u64::<LittleEndian>().unwrap()
        } else {
            self.inner.read_u32::<LittleEndian>().unwrap() as u64
        }
    }
    fn string(&mut self) -> String {
        let n = self.size() as usize;
        let mut bytes = vec![0u8; n];
        self.inner.read_exact(&mut bytes).unwrap();
        while bytes.last() == Some(&0) {
            bytes.pop(); // version-1 files may carry a terminator
        }
        String::from_utf8_lossy(&bytes).into_owned()
    }
    /// Reads one metadata value of type `t`; returns it when it is an integer of at most 32 bits.
    fn value(&mut self, t: u32) -> Option<i64> {
        let r = &mut self.inner;
        match t {
            0 => Some(r.read_u8().unwrap() as i64),
            1 => Some(r.read_i8().unwrap() as i64),
            2 => Some(r.read_u16::<LittleEndian>().unwrap() as i64),
            3 => Some(r.read_i16::<LittleEndian>().unwrap() as i64),
            4 => Some(r.read_u32::<LittleEndian>().unwrap() as i64),
            5 => Some(r.read_i32::<LittleEndian>().unwrap() as i64),
            6 => r.read_f32::<LittleEndian>().map(|_| None).unwrap(),
            7 => match r.read_u8().unwrap() {
                0 | 1 => None,
                b => panic!("unexpected bool value {b}"),
            },
            8 => {
                self.string();
                None
            }
            9 => {
                let element = self.inner.read_u32::<LittleEndian>().unwrap();
                for _ in 0..self.size() {
                    self.value(element);
                }
                None
            }
            10 | 11 => r.read_u64::<LittleEndian>().map(|_| None).unwrap(),
            12 => r.read_f64::<LittleEndian>().map(|_| None).unwrap(),
            _ => panic!("unrecognized value-type {t:#08x}"),
        }
    }
}

fn read_header<R: Read + Seek>(inner: R) -> Header {
    let mut r = Reader { inner, wide: true };
    let magic = r.inner.read_u32::<LittleEndian>().unwrap();
    assert!(magic == 0x4655_4747 || magic == 0x4747_5546, "unknown magic 0x{magic:08x}");
    let version = r.inner.read_u32::<LittleEndian>().unwrap();
    assert!((1..=3).contains(&version), "gguf: unsupported version {version}");
    r.wide = version > 1;
    let (tensor_count, kv_count) = (r.size(), r.size());
    let mut alignment = DEFAULT_ALIGNMENT;
    for _ in 0..kv_count {
        let key = r.string();
        let t = r.inner.read_u32::<LittleEndian>().unwrap();
        let v = r.value(t);
        if key == "general.alignment" {
            if let Some(a) = v.filter(|a| *a > 0) {
                alignment = a as u64;
            }
        }
    }
    let mut tensors = HashMap::new();
    for _ in 0..tensor_count {
        let name = r.string();
        let n_dims = r.inner.read_u32::<LittleEndian>().unwrap();
        let n_elements = (0..n_dims).map(|_| r.size() as usize).product::<usize>();
        let dtype = r.inner.read_u32::<LittleEndian>().unwrap();
        let offset = r.inner.read_u64::<LittleEndian>().unwrap();
        tensors.insert(name, TensorInfo { n_elements, offset, dtype });
    }
    let pos = r.inner.stream_position().unwrap();
    Header { tensors, data_offset: pos.div_ceil(alignment) * alignment }
}

/// Points every parameter of `model` at its tensor in the GGUF file and returns the nodes that hold Q8_0 weights,
/// for `HipQuantizedCompiler::new`.  The bytes are read when the graph first runs the node: F32 tensors become
/// host `Vec<f32>`, Q8_0 tensors are uploaded and re-arranged on the device into the planar form the kernels read
/// (the file's 34-byte blocks never reach a matmul).  Any other ggml dtype panics, as in the reference loader.
pub fn q8_load_hip<P: AsRef<Path>, M: SerializeModule>(path: P, model: &M, graph: &mut Graph) -> Vec<NodeIndex> {
    let Header { mut tensors, data_offset } = read_header(File::open(&path).unwrap());
    let mut q8_weights = vec![];
    for (weight_name, node_index) in param_dict(model) {
        let Some(loading_node) = graph.graph.node_weight_mut(node_index).and_then(|op| op.as_any_mut().downcast_mut::<Function>()) else {
            continue;
        };
        let file_path = path.as_ref().to_owned();
        let TensorInfo { n_elements, offset, dtype } = tensors.remove(&weight_name.replace('/', ".")).unwrap();
        let n_bytes = match dtype {
            GGML_F32 => n_elements * 4,
            GGML_Q8_0 => {
                q8_weights.push(node_index);
                n_elements + n_elements / 16
            }
            _ => panic!("Unsupported dtype: {dtype}"),
        };
        loading_node.1 = Box::new(move |_| {
            let mut bytes = vec![0u8; n_bytes];
            let mut file = File::open(&file_path).unwrap();
            file.seek(SeekFrom::Start(offset + data_offset)).unwrap();
            file.read_exact(&mut bytes).unwrap();
            match dtype {
                GGML_F32 => {
                    vec![Tensor::new(bytes.chunks_exact(4).map(|c| f32::from_le_bytes([c[0], c[1], c[2], c[3]])).collect::<Vec<f32>>())]
                }
                _ => vec![Tensor::new(HipData::q8_0_from_raw(&bytes, n_elements))],
            }
        });
    }
    q8_weights
}
