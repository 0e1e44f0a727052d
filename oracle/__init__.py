"""CPU oracle of the W4A4 linear path: TEST INFRASTRUCTURE ONLY.

quest_oracle.py restates the reference's PyTorch baseline with torch CPU ops, quest_oracle.c
restates it again as scalar C.  Nothing under quest_amd/ may import this package.
"""
